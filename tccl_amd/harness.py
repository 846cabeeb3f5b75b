"""Size sweep in the shape of the reference's ``__main__`` benchmarks.

The reference halves the message size from 256 Mi elements down to 2,048 and prints one
line per size, ``"<name> <bytes> <rate> MB/s"`` (triton_reduce_scatter.py:213-240,
triton_all_gather.py:177-204, triton_double_tree_allreduce.py:412-438); its "MB/s" is
really bytes / ms / 1e6 = GB/s of *input bytes per rank*, timed over 10 calls with no
warm-up.  This harness prints the same columns with the unit fixed (GB/s of input bytes per
rank, as the reference counts them) plus the algorithmic HBM GB/s, after a warm-up, timed
with HIP events on the launch stream.

    python -m tccl_amd.harness all_reduce|reduce_scatter|all_gather|double_tree|double_tree_pipelined|
                               two_shot|two_shot_world [--world 8] [--max-elems N] [--compare] [--plot out.png]

Started once per rank (``python -m tccl_amd.launch --nproc-per-node 8 --module tccl_amd.harness all_reduce``) it is the
reference's benchmark as the reference runs it: every rank a process of its own with its own symmetric
buffer (``tccl_amd.ipc.IpcWorld``), every call one launch per rank with the blockwise barrier inside,
rank 0 printing the lines; the operations are then ``all_reduce``, ``reduce_scatter``, ``all_gather``,
``two_shot``, ``double_tree`` and ``auto`` (``tccl_amd.all_reduce(tensor)``: the algorithm picked by size).

``--plot`` draws what the reference's notebook draws (plot.ipynb: message size against rate, both
axes logarithmic, one curve per implementation) from the lines just printed, with the axis in
GB/s as measured (the notebook multiplies its GB/s by 1e6 and calls them B/s).
"""
from __future__ import annotations

import argparse
import ctypes
import os
import sys

import re
from typing import List, Optional, Tuple

REPS = 10          # as in the reference

_LINE = re.compile(r"^(?P<name>\S+) (?P<bytes>\d+) (?P<rate>[0-9.]+(?:e[+-]?\d+)?|inf|nan) GB/s")


def parse_line(line: str) -> Optional[Tuple[str, int, float]]:
    """``"<name> <bytes> <rate> GB/s ..."`` -> (name, bytes, rate); None for any other line."""
    m = _LINE.match(line.strip())
    if not m:
        return None
    return m.group("name"), int(m.group("bytes")), float(m.group("rate"))


def plot(lines: List[str], path: str, title: str) -> None:
    """Message size against rate, both axes logarithmic, one curve per name."""
    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt
    curves = {}
    for ln in lines:
        rec = parse_line(ln)
        if rec is not None:
            curves.setdefault(rec[0], []).append(rec[1:])
    fig, ax = plt.subplots(figsize=(7, 4.5))
    for name, pts in curves.items():
        pts.sort()
        ax.plot([p[0] for p in pts], [p[1] for p in pts], marker="o", markersize=3, label=name)
    ax.set_xscale("log", base=2)
    ax.set_yscale("log")
    ax.set_xlabel("input bytes per rank")
    ax.set_ylabel("GB/s of input bytes per rank")
    ax.set_title(title)
    ax.grid(True, which="both", linewidth=0.3)
    ax.legend()
    fig.tight_layout()
    fig.savefig(path, dpi=120)
    plt.close(fig)


def per_rank_main(args) -> int:
    """This process is one rank (started by ``python -m tccl_amd.launch``): the reference's benchmark loop
    (triton_reduce_scatter.py:213-240) on this rank's symmetric buffer, the peers being other processes."""
    import torch
    import tccl_amd
    from tccl_amd import ipc
    world = ipc.IpcWorld.from_env()
    rank, size = world.rank, world.world_size
    ops = {
        "all_reduce": (tccl_amd.one_shot_all_reduce, lambda n: (size + 1) * n * 2),
        "reduce_scatter": (tccl_amd.reduce_scatter, lambda n: (size + 1) * (n // size) * 2),
        "all_gather": (lambda t: tccl_amd.all_gather(t, size), lambda n: 2 * size * n * 2),
        "two_shot": (tccl_amd.two_shot_all_reduce, lambda n: (3 * size - 1) * (n // size) * 2),
        "double_tree": (tccl_amd.double_tree_all_reduce, None),
        "auto": (tccl_amd.all_reduce, None),
    }
    if args.op not in ops:
        if rank == 0:
            print(f"{args.op} runs every rank's work from one process; with a process per rank use one of {sorted(ops)}",
                  file=sys.stderr)
        world.close()
        return 2
    fn, algo_bytes = ops[args.op]
    max_elems = args.max_elems // (8 * size) * (8 * size)
    tensor = world.empty(max_elems, torch.bfloat16)
    torch.manual_seed(rank)
    tensor.copy_(torch.randn(1 << 16, dtype=torch.bfloat16).repeat(-(-max_elems // (1 << 16)))[:max_elems] * (1.0 / 64))
    in_place = args.op in ("two_shot", "double_tree", "auto")
    printed: List[str] = []
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n = max_elems
    while n >= 2048:
        n = n // (8 * size) * (8 * size)
        view = tensor[:n]
        fn(view)                                    # warm-up (the reference has none)
        start.record()
        for _ in range(REPS):
            if in_place:
                view.mul_(1.0 / size)               # an in-place sum over and over would run away; part of the time
            fn(view)
        stop.record()
        stop.synchronize()
        world.check()
        per_call_ms = start.elapsed_time(stop) / REPS
        if rank == 0:
            line = f"tccl_amd {n * 2} {n * 2 / per_call_ms / 1e6:.3f} GB/s"
            if algo_bytes is not None:
                line += f"  (HBM {algo_bytes(n) / per_call_ms / 1e6:.1f} GB/s for this rank, {per_call_ms * 1e3:.1f} us)"
            else:
                line += f"  ({per_call_ms * 1e3:.1f} us" + (f", {world.auto_algorithm(view)})" if args.op == "auto" else ")")
            printed.append(line)
            print(line, flush=True)
        n //= 2
    world.close()
    if rank == 0 and args.plot:
        plot(printed, args.plot, f"{args.op}, {size} processes (one rank each) on one MI355X")
        print(f"plot written to {args.plot}", flush=True)
    return 0


def main(argv=None) -> int:
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("op", choices=["all_reduce", "reduce_scatter", "all_gather", "double_tree", "double_tree_plan", "double_tree_fused",
                                  "double_tree_pipelined", "two_shot", "two_shot_world", "auto"])
    p.add_argument("--world", type=int, default=8)
    p.add_argument("--max-elems", type=int, default=256 * 1024 * 1024 // 2,
                   help="largest element count per rank (bf16); halved down to 2,048")
    p.add_argument("--plot", metavar="PNG", help="also draw the curves (log-log, GB/s) into this file")
    p.add_argument("--compare", action="store_true",
                   help="also time the same operation written with torch's own GPU kernels, as the second "
                        "line per size (the place the reference gives to NCCL)")
    args = p.parse_args(argv)
    if "RANK" in os.environ and "TCCL_RENDEZVOUS_DIR" in os.environ:
        return per_rank_main(args)
    if args.op == "auto":
        p.error("auto is an operation of the per-rank form (start the harness through python -m tccl_amd.launch)")

    import torch
    import tccl_amd
    lib = tccl_amd.load_library()
    world = args.world
    group = tccl_amd.empty_world(world, args.max_elems, torch.bfloat16, "cuda")
    for r in range(world):
        torch.manual_seed(r)
        group.tensor(r).normal_()
    tensor = group.tensor(min(3, world - 1))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    start, stop = ctypes.c_void_p(), ctypes.c_void_p()
    lib.tccl_event_create(ctypes.byref(start))
    lib.tccl_event_create(ctypes.byref(stop))

    fns = {
        "all_reduce": (tccl_amd.one_shot_all_reduce, lambda n: (world + 1) * n * 2),
        "two_shot": (tccl_amd.two_shot_all_reduce, lambda n: (world + 3) * n * 2),
        "reduce_scatter": (tccl_amd.reduce_scatter, lambda n: (world + 1) * (n // world) * 2),
        "all_gather": (lambda t: tccl_amd.all_gather(t, world), lambda n: 2 * world * n * 2),
        "double_tree": (lambda t: tccl_amd.double_tree_all_reduce_world(group, t.numel(), fused=False, pipelined=False),
                        None),
        "double_tree_fused": (lambda t: tccl_amd.double_tree_all_reduce_world(group, t.numel(), fused=True), None),
        # one persistent launch, virtual ranks signalling each other per chunk
        "double_tree_pipelined": (lambda t: tccl_amd.double_tree_all_reduce_world(group, t.numel(), pipelined=True),
                                  None),
        # every rank's all-reduce in place in one launch (reduce own share, barrier, gather the rest)
        "two_shot_world": (lambda t: tccl_amd.two_shot_all_reduce_world(group, t.numel(), with_outputs=False),
                           lambda n: (3 * world - 1) * n * 2),
    }

    def torch_eager(view):
        """The operation with torch's stock kernels on the same buffers (fp32 accumulate)."""
        n = view.numel()
        srcs = [group.tensor(r)[:n] for r in range(world)]
        if args.op == "all_gather":
            return torch.stack(srcs)
        if args.op == "reduce_scatter":
            per = n // world
            r = min(3, world - 1)
            srcs = [b[r * per:(r + 1) * per] for b in srcs]
        acc = srcs[0].float()
        for b in srcs[1:]:
            acc += b
        return acc.to(view.dtype)

    printed: List[str] = []

    def emit(line: str) -> None:
        printed.append(line)
        print(line, flush=True)

    size = args.max_elems
    while size >= 2048:
        size = size // (8 * world) * (8 * world)     # whole 16-byte vectors per rank share, whatever --max-elems was
        view = tensor[:size]
        if args.op == "double_tree_plan":       # one recorded plan per size, replayed
            plan = tccl_amd.DoubleTreePlan(group, size)
            fn, algo_bytes = (lambda t: plan.run()), None
        else:
            fn, algo_bytes = fns[args.op]
        fn(view)                                    # warm-up (the reference has none)
        lib.tccl_event_record(start, stream)
        for _ in range(REPS):
            fn(view)
        lib.tccl_event_record(stop, stream)
        lib.tccl_event_synchronize(stop)
        ms = ctypes.c_float()
        lib.tccl_event_elapsed_ms(start, stop, ctypes.byref(ms))
        per_call_ms = ms.value / REPS
        line = f"tccl_amd {size * 2} {size * 2 / per_call_ms / 1e6:.3f} GB/s"
        if algo_bytes is not None:
            line += f"  (HBM {algo_bytes(size) / per_call_ms / 1e6:.1f} GB/s, {per_call_ms * 1e3:.1f} us)"
        else:
            line += f"  ({per_call_ms * 1e3:.1f} us)"
        emit(line)
        if args.compare:
            torch_eager(view)
            lib.tccl_event_record(start, stream)
            for _ in range(REPS):
                torch_eager(view)
            lib.tccl_event_record(stop, stream)
            lib.tccl_event_synchronize(stop)
            lib.tccl_event_elapsed_ms(start, stop, ctypes.byref(ms))
            t_ms = ms.value / REPS
            emit(f"torch {size * 2} {size * 2 / t_ms / 1e6:.3f} GB/s  ({t_ms * 1e3:.1f} us)")
        size //= 2
    if args.op in ("double_tree_pipelined", "two_shot_world"):
        expired = tccl_amd.signal_pad_timeouts(group)
        print(f"expired waits: {expired}", flush=True)
    tccl_amd.unregister(group)
    if args.plot:
        plot(printed, args.plot, f"{args.op}, {world} virtual ranks on one MI355X")
        print(f"plot written to {args.plot}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
