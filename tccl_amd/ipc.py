"""Symmetric buffers owned by separate processes on one GPU.

The reference's ranks are processes: each allocates its buffer with
``_SymmetricMemory.empty_strided_p2p`` (triton_one_shot_all_reduce_no_128.py:116-122) and gets
the table of all ranks' buffer addresses from ``rendezvous`` (:82).  This module does the same
for W processes that share one MI355X: a rank's buffer is a device allocation of its own
(``tccl_symm_alloc``), exported as a 64-byte handle, carried to the peers through a directory
they all see, and mapped there (``tccl_ipc_open``).  The resulting ``SymmHandle`` goes through
the same wrappers as a group of virtual ranks (``one_shot_all_reduce``, ``reduce_scatter``,
``all_gather``); ordering between the ranks' launches is the reference's device-side
``blockwise_barrier`` (triton_barrier.py:39-142) inside the collective's kernel, as the reference
has it (triton_one_shot_all_reduce_no_128.py:46), before the first read and -- what the reference
lacks -- after the last one: a collective is one launch per rank, and when it has ended on a
rank's stream that rank may refill its buffer.  (Large one-shot inputs run as barrier launch, the
full-size kernel, barrier launch instead: ``IpcWorld.FUSED_MAX_MOVED_BYTES``.)

    world = IpcWorld(rank, world_size, directory)          # one per process
    tensor = world.empty(numel, torch.bfloat16)            # this rank's buffer, peers mapped
    tensor.copy_(...)
    out = tccl_amd.one_shot_all_reduce(tensor)             # waits for the peers' buffers itself
    world.check()                                          # raises if a wait inside a kernel expired
    world.close()

``IpcWorld.barrier`` is the barrier alone (one launch per rank), ``IpcWorld.all_reduce`` picks
between the one-shot, two-shot and double-tree forms by size, ``IpcWorld.reset`` clears the pads
after a time-out.
"""
from __future__ import annotations

import ctypes
import os
import time
from typing import List, Optional

import torch

from . import _lib, symm

_DTYPE_TYPESTR = {torch.bfloat16: None, torch.float32: "<f4", torch.int8: "|i1", torch.uint8: "|u1", torch.int16: "<i2",
                  torch.int32: "<i4"}


class _DeviceBlock:
    """A raw device allocation seen through ``__cuda_array_interface__`` so that torch can wrap it."""

    def __init__(self, ptr: int, nbytes: int):
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (ptr, False), "version": 2}


def _as_tensor(ptr: int, nbytes: int, device) -> torch.Tensor:
    return torch.as_tensor(_DeviceBlock(ptr, nbytes), device=device)


def _refuse_used_directory(directory: str, rank: int) -> None:
    """The handle files have fixed names (``pad0.rank3``, ``buf1.rank0`` ...): in a directory that an
    earlier run has used, this run's ranks would read that run's 64-byte handles and try to map
    allocations that no longer exist.  A rank therefore refuses a directory that already holds a file
    of its own rank (every rank writes before it reads, so in a fresh directory none can exist yet)."""
    suffix = f".rank{rank}"
    try:
        names = os.listdir(directory)
    except OSError as e:
        raise RuntimeError(f"the rendezvous directory {directory!r} cannot be read: {e}") from None
    old = sorted(n for n in names if n.endswith(suffix) or n.endswith(f".tmp{rank}"))
    if old:
        raise RuntimeError(f"the rendezvous directory {directory!r} already holds files of rank {rank} from another run "
                           f"({', '.join(old[:3])}{' ...' if len(old) > 3 else ''}): every run needs a fresh directory "
                           "(python -m tccl_amd.launch makes one)")


class IpcWorld:
    """This process's view of W processes sharing one GPU.  ``directory`` is where the ranks leave
    their handles for each other (any place all of them can read and write)."""

    BARRIER_BLOCKS = 4
    PAD_BYTES = 4096

    def __init__(self, rank: int, world_size: int, directory: str, device="cuda:0", timeout_s: float = 60.0):
        if not (1 <= world_size <= _lib.MAX_WORLD and 0 <= rank < world_size):
            raise ValueError("rank/world_size out of range")
        self.rank, self.world_size, self.directory, self.timeout_s = rank, world_size, directory, timeout_s
        _refuse_used_directory(directory, rank)
        self.device = torch.device(device)
        self.lib = _lib.load()
        self._allocs: List[int] = []          # own allocations
        self._opened: List[int] = []          # peers' allocations mapped here
        self._tables = {}                     # own buffer address -> (all ranks' addresses, bytes, dtype)
        self._family_pads = {}                  # (kernel family, pad size) -> table of all ranks' pads for kernels that signal inside a launch
        self._count = 0
        self._host_barriers = 0
        self._epoch = 0                       # resets so far: time-outs are published per epoch
        self._flag = ctypes.POINTER(ctypes.c_uint32)()
        _lib.check("tccl_timeout_flag_create", self.lib.tccl_timeout_flag_create(ctypes.byref(self._flag)))
        # signal pads: one per rank, every rank maps all of them
        self._pad_ptrs = self._exchange(self._alloc(self.PAD_BYTES), "pad")
        self._pad_array = _lib.ptr_array(self._pad_ptrs)
        # ... and the pads of the one-shot and two-shot kernels that carry their barriers themselves, so that
        # a rank's first collective never has to wait on the host for a peer that is late (the double tree's
        # pads depend on the input's size and are made when a size is first used)
        self._kernel_pads(self.ONE_SHOT_PAD_BYTES, "one_shot")
        self._kernel_pads(self.TWO_SHOT_PAD_BYTES, "two_shot")

    @classmethod
    def from_env(cls, device="cuda:0", timeout_s: float = 60.0) -> "IpcWorld":
        """The world a launcher describes in the environment, as the reference's programs read it
        (triton_one_shot_all_reduce_no_128.py:106-108): RANK and WORLD_SIZE, plus
        TCCL_RENDEZVOUS_DIR, the directory the ranks exchange their handles through
        (``python -m tccl_amd.launch`` sets all three)."""
        try:
            rank, world_size = int(os.environ["RANK"]), int(os.environ["WORLD_SIZE"])
            directory = os.environ["TCCL_RENDEZVOUS_DIR"]
        except KeyError as e:
            raise RuntimeError(f"{e.args[0]} is not set: start the program with python -m tccl_amd.launch") from None
        return cls(rank, world_size, directory, device=device, timeout_s=timeout_s)

    # ---- plumbing
    def _alloc(self, nbytes: int) -> int:
        p = ctypes.c_void_p()
        _lib.check("tccl_symm_alloc", self.lib.tccl_symm_alloc(nbytes, ctypes.byref(p)))
        self._allocs.append(p.value)
        return p.value

    def _wait_for(self, path: str) -> bytes:
        t_end = time.monotonic() + self.timeout_s
        while time.monotonic() < t_end:
            try:
                with open(path, "rb") as f:
                    data = f.read()
                if data:
                    return data
            except OSError:
                pass
            time.sleep(0.002)
        raise TimeoutError(f"rank {self.rank}: {path} did not appear within {self.timeout_s} s")

    def _publish(self, name: str, data: bytes) -> None:
        tmp = os.path.join(self.directory, f".{name}.tmp{self.rank}")
        with open(tmp, "wb") as f:
            f.write(data)
        os.replace(tmp, os.path.join(self.directory, name))          # appears whole or not at all

    def _exchange(self, own_ptr: int, what: str) -> List[int]:
        """Export own_ptr, collect everybody's handle, map the peers'; addresses in rank order."""
        tag = f"{what}{self._count}"
        self._count += 1
        handle = (ctypes.c_ubyte * _lib.IPC_HANDLE_BYTES)()
        _lib.check("tccl_ipc_export", self.lib.tccl_ipc_export(own_ptr, handle))
        self._publish(f"{tag}.rank{self.rank}", bytes(handle))
        ptrs = []
        for r in range(self.world_size):
            if r == self.rank:
                ptrs.append(own_ptr)
                continue
            raw = self._wait_for(os.path.join(self.directory, f"{tag}.rank{r}"))
            h = (ctypes.c_ubyte * _lib.IPC_HANDLE_BYTES).from_buffer_copy(raw)
            p = ctypes.c_void_p()
            _lib.check("tccl_ipc_open", self.lib.tccl_ipc_open(h, ctypes.byref(p)))
            self._opened.append(p.value)
            ptrs.append(p.value)
        return ptrs

    # ---- what a per-rank program uses
    def empty(self, numel: int, dtype: torch.dtype) -> torch.Tensor:
        """This rank's buffer of a symmetric allocation (zero-filled), registered with the peers'
        mapped buffers as one group: collective, every rank must make the same calls in the same
        order (as with ``empty_strided_p2p`` followed by ``rendezvous``)."""
        esize = torch.empty(0, dtype=dtype).element_size()
        nbytes = numel * esize
        own = self._alloc(max(nbytes, 16))
        ptrs = self._exchange(own, "buf")
        tensor = _as_tensor(own, nbytes, self.device).view(dtype)
        symm.register_remote(tensor, self.rank, ptrs, world=self)
        self._tables[own] = (ptrs, nbytes, dtype)
        return tensor

    def peers(self, tensor: torch.Tensor) -> List[torch.Tensor]:
        """All ranks' buffers of the symmetric allocation ``tensor`` came from, in rank order (this
        rank's own at index ``rank``), as tensors over the mapped memory: what the reference gets
        from ``symm_mem.get_buffer(rank, ...)``.  Reading a peer's buffer is ordered against the
        peer's writes by ``barrier()`` like everything else."""
        ptrs, nbytes, dtype = self._tables[self._base(tensor)]
        return [_as_tensor(p, nbytes, self.device).view(dtype) for p in ptrs]

    def host_barrier(self) -> None:
        """All ranks have reached this point on the host (through the directory)."""
        tag = f"host{self._host_barriers}"
        self._host_barriers += 1
        self._publish(f"{tag}.rank{self.rank}", b"1")
        for r in range(self.world_size):
            self._wait_for(os.path.join(self.directory, f"{tag}.rank{r}"))

    def barrier(self, spin_limit: int = 0, blocks: Optional[int] = None) -> None:
        """The reference's ``blockwise_barrier`` on torch's current stream: everything this rank
        enqueued before is complete before any rank's later work starts.  Asynchronous; a wait
        that expires is reported by ``check()``.  ``blocks``: rows of slots used (the reference's
        own test launches 32, triton_barrier.py:155-160); every rank must pass the same."""
        stream = ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
        rc = self.lib.tccl_blockwise_barrier(self._pad_array, self.PAD_BYTES, self.world_size, self.rank,
                                             self.BARRIER_BLOCKS if blocks is None else blocks, spin_limit, self._flag,
                                             stream)
        _lib.check("tccl_blockwise_barrier", rc)

    def signal_pad(self) -> torch.Tensor:
        """This rank's signal pad as a tensor of 32-bit words (what the reference prints after its
        barrier test, triton_barrier.py:178-190): all zero whenever no barrier is running."""
        return _as_tensor(self._pad_ptrs[self.rank], self.PAD_BYTES, self.device).view(torch.int32)

    # Signal pad size the two-shot kernel is given: room for 1024 workgroups per rank.
    TWO_SHOT_PAD_BYTES = 4 * (8 * 1024 + 288)

    def _kernel_pads(self, nbytes: int, family: str) -> ctypes.Array:
        """All ranks' signal pads of `nbytes` for the kernels of one family ("one_shot", "two_shot",
        "double_tree") that signal inside a launch (collective on first use, like ``empty``).  Every
        family has pads of its own: each lays its barrier rows out differently, and a kernel that ends
        while a slower peer has yet to take its last flags may only be followed, on the same pads, by a
        kernel that keeps those rows for the same purpose."""
        key = (family, nbytes)
        if key not in self._family_pads:
            self._family_pads[key] = _lib.ptr_array(self._exchange(self._alloc(nbytes), "kpad"))
        return self._family_pads[key]

    def _own_launch(self, name: str, family: str, tensor: torch.Tensor, pad_bytes: int, tail_args, cfg,
                    own_barriers: bool = False) -> torch.Tensor:
        ptrs, _, dtype = self._tables[self._base(tensor)]
        code = {torch.bfloat16: _lib.TCCL_BF16, torch.float32: _lib.TCCL_F32}[dtype]
        pads = self._kernel_pads(pad_bytes, family)
        use = _lib.PipelineCfg()
        if cfg is not None:
            ctypes.memmove(ctypes.byref(use), ctypes.byref(cfg), ctypes.sizeof(use))
        use.timeout_flag = self._flag
        if own_barriers:
            use.flags |= _lib.PIPE_OWN_BARRIERS            # the kernel begins and ends with the barrier itself
        out = torch.empty_like(tensor)
        stream = ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
        if not own_barriers:
            self.barrier()                                 # every rank's input is in place
        rc = getattr(self.lib, name)(_lib.ptr_array(ptrs), out.data_ptr(), pads, pad_bytes, self.world_size, self.rank,
                                     tensor.numel(), code, *tail_args, ctypes.byref(use), stream)
        _lib.check(name, rc)
        if not own_barriers:
            self.barrier()                                 # every rank is done with buffers and pads
        return out

    def double_tree_all_reduce(self, tensor: torch.Tensor, chunk_elems: int = 0,
                               cfg: Optional[_lib.PipelineCfg] = None, own_barriers: bool = True) -> torch.Tensor:
        """The reference's double-tree all-reduce as it runs it (triton_double_tree_allreduce.py:338-370):
        this rank's own launch of the pipelined kernel, meeting the other ranks' launches through
        wait/send on signal pads in each other's memory; the kernel begins with the blockwise barrier
        as the reference's does (:239) and ends with one (``own_barriers=False``: a barrier launch
        before and after instead).  Collective; the symmetric buffers are overwritten (every rank's
        ends up holding the sum, which is also returned).  Worlds of 2, 4 and 8."""
        _, _, dtype = self._tables[self._base(tensor)]
        code = {torch.bfloat16: _lib.TCCL_BF16, torch.float32: _lib.TCCL_F32}[dtype]
        need = self.lib.tccl_double_tree_signal_pad_bytes(self.world_size, tensor.numel(), code, chunk_elems)
        if need == 0:
            raise ValueError("the pipelined double tree takes worlds of 2, 4 or 8 and whole 16-byte vectors")
        if tensor.numel() == 0:
            return torch.empty_like(tensor)
        return self._own_launch("tccl_double_tree_all_reduce_pipelined_rank", "double_tree", tensor, need, (chunk_elems,), cfg, own_barriers)

    def two_shot_all_reduce(self, tensor: torch.Tensor, cfg: Optional[_lib.PipelineCfg] = None,
                            own_barriers: bool = True) -> torch.Tensor:
        """Two-shot all-reduce, this rank's own launch: reduce the own share from all buffers, meet
        the other ranks' kernels in the reference's blockwise barrier (triton_barrier.py:39-142,
        inside the kernel, as the reference uses it), gather the other shares.  Collective, in
        place (every buffer ends up holding the sum, which is also returned); bit-identical to
        ``one_shot_all_reduce``.  The element count must be a multiple of W vectors.
        ``own_barriers``: the kernel also begins and ends with that barrier (one launch per rank);
        False = a barrier launch before and after instead."""
        if tensor.numel() == 0:
            return torch.empty_like(tensor)
        return self._own_launch("tccl_two_shot_all_reduce_rank", "two_shot", tensor, self.TWO_SHOT_PAD_BYTES, (), cfg, own_barriers)

    # Signal pad size of the one-shot kernels: two rows of slots for up to 512 workgroups per rank.
    ONE_SHOT_PAD_BYTES = 4 * (2 * 8 * 512 + 288)

    # A one-shot collective is ONE launch with the barriers inside while its kernel moves at most this many
    # bytes, and barrier launch + the library's full-size kernel + barrier launch above: a rank's own launch
    # holds only 1/W of the workgroups that are certain to find room beside the peers' launches and works in
    # 16 KiB tiles, which costs more than two extra launches once the data is large (8 processes on one
    # MI355X, all-reduce of 8 x 16 MiB = 144 MiB moved: 292-298 us fused against 290-345 us; 8 x 64 MiB:
    # 1,024-1,114 against 871-915 us; reduce-scatter of 8 x 256 MiB = 288 MiB moved: 526-559 against 463-521 us, of
    # 8 x 64 MiB = 72 MiB: 172-175 against 200-250 us; profiles/ipc_forms_one_gpu_8_4_2_processes.txt).
    FUSED_MAX_MOVED_BYTES = 128 << 20

    def _one_shot(self, name: str, tensor: torch.Tensor, out: torch.Tensor, size_arg: int, with_dtype: bool,
                  cfg: Optional[_lib.PipelineCfg], moved_bytes: int = 0, fused: Optional[bool] = None) -> torch.Tensor:
        ptrs, _, dtype = self._tables[self._base(tensor)]
        if fused is None:
            fused = moved_bytes <= self.FUSED_MAX_MOVED_BYTES
        if not fused:
            if cfg is not None:
                raise ValueError("a PipelineCfg applies to the one-launch form only (fused=True)")
            stream = ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
            plain = name[:-len("_rank")]
            args = [_lib.ptr_array(ptrs), self.world_size]
            if plain == "tccl_reduce_scatter_sum":
                args.append(self.rank)
            args += [out.data_ptr(), size_arg]
            if with_dtype:
                args.append({torch.bfloat16: _lib.TCCL_BF16, torch.float32: _lib.TCCL_F32}[dtype])
            self.barrier()                                     # every rank's input is in place
            _lib.check(plain, getattr(self.lib, plain)(*args, stream))
            self.barrier()                                     # every rank has read every buffer
            return out
        pads = self._kernel_pads(self.ONE_SHOT_PAD_BYTES, "one_shot")
        use = _lib.PipelineCfg()
        if cfg is not None:
            ctypes.memmove(ctypes.byref(use), ctypes.byref(cfg), ctypes.sizeof(use))
        use.timeout_flag = self._flag
        stream = ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
        args = [_lib.ptr_array(ptrs), out.data_ptr(), pads, self.ONE_SHOT_PAD_BYTES, self.world_size, self.rank, size_arg]
        if with_dtype:
            args.append({torch.bfloat16: _lib.TCCL_BF16, torch.float32: _lib.TCCL_F32}[dtype])
        _lib.check(name, getattr(self.lib, name)(*args, ctypes.byref(use), stream))
        return out

    def _base(self, tensor: torch.Tensor) -> int:
        """Address of the symmetric buffer ``tensor`` is (a prefix view of)."""
        base = tensor.data_ptr()
        if base not in self._tables:
            raise RuntimeError("tensor does not come from this world's empty() (or is not a view from its first element)")
        if not tensor.is_contiguous():
            raise RuntimeError("a collective must be given a contiguous view")
        return base

    def one_shot_all_reduce(self, tensor: torch.Tensor, *, out: Optional[torch.Tensor] = None,
                            cfg: Optional[_lib.PipelineCfg] = None, fused: Optional[bool] = None) -> torch.Tensor:
        """``one_shot_all_reduce`` the way the reference's kernel runs it (triton_one_shot_all_reduce_no_128.py:35-64):
        this rank's ONE launch, which meets the peers' launches in ``blockwise_barrier`` first (:46), sums all
        W buffers in rank order into a fresh output, and meets the peers again before it ends (so the buffers
        may be refilled as soon as the call's kernel is done).  Collective: every rank calls it.
        ``fused``: None = that form up to ``FUSED_MAX_MOVED_BYTES``, above it a barrier launch, the
        library's full-size kernel and a barrier launch (same values, same guarantees); True / False force one."""
        assert tensor.dtype in (torch.bfloat16, torch.float32), "Only bfloat16 (and float32) is supported for now."
        assert tensor.numel() % (16 // tensor.element_size()) == 0, "The number of elements must be 128-bit aligned."
        output = torch.empty_like(tensor) if out is None else out
        moved = (self.world_size + 1) * tensor.numel() * tensor.element_size()
        return self._one_shot("tccl_all_reduce_sum_rank", tensor, output, tensor.numel(), True, cfg, moved, fused)

    def reduce_scatter(self, tensor: torch.Tensor, *, out: Optional[torch.Tensor] = None,
                       cfg: Optional[_lib.PipelineCfg] = None, fused: Optional[bool] = None) -> torch.Tensor:
        """``one_shot_reduce_scatter`` as one launch of this rank with the barriers inside the kernel
        (triton_reduce_scatter.py:59-92; the reference has its leading barrier commented out, :70)."""
        assert tensor.dtype in (torch.bfloat16, torch.float32), "Only bfloat16 (and float32) is supported for now."
        assert tensor.numel() % ((16 // tensor.element_size()) * self.world_size) == 0, \
            "The number of elements must be 128-bit aligned."
        per_rank = tensor.numel() // self.world_size
        output = torch.empty((per_rank,), dtype=tensor.dtype, device=tensor.device) if out is None else out
        moved = (self.world_size + 1) * per_rank * tensor.element_size()
        return self._one_shot("tccl_reduce_scatter_sum_rank", tensor, output, tensor.numel(), True, cfg, moved, fused)

    def all_gather(self, tensor: torch.Tensor, *, out: Optional[torch.Tensor] = None,
                   cfg: Optional[_lib.PipelineCfg] = None, fused: Optional[bool] = None) -> torch.Tensor:
        """``one_shot_all_gather`` as one launch of this rank with the barriers inside the kernel
        (triton_all_gather.py:32-63, leading barrier :43)."""
        nbytes = tensor.numel() * tensor.element_size()
        assert nbytes % 16 == 0, "The number of elements must be 128-bit aligned."
        if out is None:
            out = torch.empty((self.world_size, *tensor.shape), dtype=tensor.dtype, device=tensor.device)
        return self._one_shot("tccl_all_gather_rank", tensor, out, nbytes, False, cfg, 2 * self.world_size * nbytes, fused)

    # all_reduce(algorithm="auto"): one-shot up to this many bytes per buffer, two-shot above it in worlds of more
    # than 4.  Measured with 8 processes on one MI355X (python -m tccl_amd.launch --nproc-per-node 8
    # benchlib/ipc_forms.py, us per collective, one-shot / two-shot / double tree; profiles/
    # ipc_forms_one_gpu_8_4_2_processes.txt): 1 MiB 59-73 / 141-186 / 167-213; 4 MiB 104-122 / 162-226 / 196-242;
    # 16 MiB 290-345 / 247-310 / 282-327; 64 MiB 871-915 / 705-765 / 834-880; 256 MiB 3,300 / 2,759-2,826 /
    # 3,140-3,211.  With 4 processes (and with 2) the one-shot form is the fastest at every size: 64 MiB
    # 206-245 / 272 / 317, 256 MiB 863 / 1,232 / 1,227; worlds of 5 to 7 were not measured and take the rule
    # of 8.  The double tree is never the fastest on one GPU and is run by name only.  Across GPUs the
    # one-shot form moves W - 1 whole buffers per rank over the links and the thresholds would sit far lower.
    ONE_SHOT_MAX_BYTES = 8 << 20
    TWO_SHOT_MIN_WORLD = 5

    def auto_algorithm(self, tensor: torch.Tensor) -> str:
        """What ``all_reduce(tensor, "auto")`` runs."""
        nbytes = tensor.numel() * tensor.element_size()
        vec = 16 // tensor.element_size()
        if nbytes > self.ONE_SHOT_MAX_BYTES and self.world_size >= self.TWO_SHOT_MIN_WORLD \
                and tensor.numel() % (vec * self.world_size) == 0:
            return "two_shot"
        return "one_shot"

    def all_reduce(self, tensor: torch.Tensor, algorithm: str = "auto") -> torch.Tensor:
        """All-reduce of this rank's buffer by the named algorithm -- ``"one_shot"`` (fresh output, buffers
        untouched), ``"two_shot"`` or ``"double_tree"`` (both in place: every buffer ends up holding the
        result, which is also returned) -- or ``"auto"``: the fastest of the three for the buffer's size and the world's (``auto_algorithm``; note
        that it may work in place)."""
        if algorithm == "auto":
            algorithm = self.auto_algorithm(tensor)
        if algorithm == "one_shot":
            return self.one_shot_all_reduce(tensor)
        if algorithm == "two_shot":
            return self.two_shot_all_reduce(tensor)
        if algorithm == "double_tree":
            return self.double_tree_all_reduce(tensor)
        raise ValueError(f"unknown all-reduce algorithm {algorithm!r}")

    def _peer_timeouts(self) -> List[int]:
        """Ranks that have published an expired wait since the last reset."""
        prefix = f"timeout{self._epoch}.rank"
        try:
            return sorted(int(n[len(prefix):]) for n in os.listdir(self.directory) if n.startswith(prefix))
        except OSError:
            return []

    def check(self) -> None:
        """Synchronise and raise if a wait of this rank expired (a peer never arrived at a barrier, or at a
        wait inside a collective's kernel), or if a peer has reported one since the last ``reset()``: that
        collective's results are partial on some rank.  Every rank should then call ``reset()``."""
        torch.cuda.synchronize(self.device)
        if self._flag[0] != 0:
            self._flag[0] = 0
            self._publish(f"timeout{self._epoch}.rank{self.rank}", b"1")
            raise _lib.TcclError("tccl_blockwise_barrier", _lib.TCCL_ETIMEOUT,
                                 "a peer did not reach the barrier in time (or a wait inside a collective's kernel expired)")
        peers = [r for r in self._peer_timeouts() if r != self.rank]
        if peers:
            raise _lib.TcclError("a collective of this world", _lib.TCCL_ETIMEOUT,
                                 f"rank(s) {peers} reported an expired wait: results since the last check may be "
                                 "partial; every rank must call reset()")

    def reset(self) -> None:
        """Collective: bring every signal pad of this world back to zero after a wait expired (a barrier
        or a signalling kernel that gave up leaves flags standing).  Every rank calls it; the ranks meet on the host before and
        after, so no barrier kernel is running while the pads are cleared."""
        torch.cuda.synchronize(self.device)
        self.host_barrier()
        _as_tensor(self._pad_ptrs[self.rank], self.PAD_BYTES, self.device).zero_()
        # the pads of the kernels that signal inside a launch, control words included: a wait that
        # expired there leaves flags standing that the next collective would take for its own
        for (_, nbytes), table in self._family_pads.items():
            _as_tensor(table[self.rank], nbytes, self.device).zero_()
        torch.cuda.synchronize(self.device)
        self._flag[0] = 0
        self._epoch += 1
        self.host_barrier()

    def close(self) -> None:
        """Unmap the peers' buffers and free the own ones (after a last host barrier, so that nobody
        unmaps what a peer is still using)."""
        torch.cuda.synchronize(self.device)
        self.host_barrier()
        for p in self._opened:
            self.lib.tccl_ipc_close(p)
        self._opened = []
        self.host_barrier()
        for p in self._allocs:
            self.lib.tccl_symm_free(p)
        self._allocs = []
        self._tables = {}
        if self._flag:
            self.lib.tccl_timeout_flag_destroy(self._flag)
            self._flag = ctypes.POINTER(ctypes.c_uint32)()
