"""What the collectives cost when every rank is a process of its own on the one GPU, form by form:

    python -m tccl_amd.launch --nproc-per-node 8 benchlib/ipc_forms.py [--json] [--sizes KiB,KiB,...]

Per buffer size rank 0 prints the time per collective (HIP events on its own stream, all ranks in
step: the median and, in brackets, the fastest of 5 blocks of 16 calls after 8 warm-up calls) of

  barrier             tccl_blockwise_barrier alone (one launch per rank)
  one-shot x3         barrier launch + tccl_all_reduce_sum + barrier launch (three launches per rank)
  one-shot fused      tccl_all_reduce_sum_rank: one launch per rank, both barriers inside the kernel
  rs x3 / rs fused    the same two forms of the reduce-scatter
  ag x3 / ag fused    ... and of the all-gather (every rank contributes 1/W of the buffer size)
  two-shot x3 / fused barrier + tccl_two_shot_all_reduce_rank + barrier, and the same kernel with
                      TCCL_PIPE_OWN_BARRIERS: one launch per rank (both in place)
  tree x3 / fused     the same two forms of tccl_double_tree_all_reduce_pipelined_rank (in place)

The in-place forms rescale the buffer before every call so that values stay finite; that small
kernel is part of their time.  On one GPU the W processes' queues take turns, so these times say how
the forms compare with each other here, not what they would cost with a GPU per rank.
``--json``: one JSON line per size instead of the table (bench.py reads those); ``--sizes``: buffer sizes
in KiB instead of 64 KiB ... 256 MiB.
``--timeline``: instead of all that, 40 barrier launches per rank, each between two one-lane kernels that store
the GPU's wall clock (benchlib/probe.hip), and rank 0 prints when every rank's stream reached each barrier and when
it left it, on that common clock: who the others wait for, and for how long."""
import ctypes
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from tccl_amd import _lib, ipc        # noqa: E402


COLUMNS = ("barrier", "one_shot_x3", "one_shot_fused", "reduce_scatter_x3", "reduce_scatter_fused", "all_gather_x3",
           "all_gather_fused", "two_shot_x3", "two_shot_fused", "double_tree_x3", "double_tree_fused")


def timeline(world) -> int:
    """When each rank's stream reaches a barrier and when it leaves it, on the GPU's one wall clock."""
    import numpy as np
    from benchlib import probe
    plib = probe.load()
    rank, size, rounds = world.rank, world.world_size, 40
    stamps = torch.zeros(2 * rounds, dtype=torch.int64, device=world.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for _ in range(8):
        world.barrier()
    torch.cuda.synchronize()
    world.host_barrier()
    for i in range(rounds):
        assert plib.tccl_probe_stamp(stamps.data_ptr() + 16 * i, stream) == 0
        world.barrier()
        assert plib.tccl_probe_stamp(stamps.data_ptr() + 16 * i + 8, stream) == 0
    torch.cuda.synchronize()
    world.check()
    np.save(os.path.join(world.directory, f"timeline.rank{rank}.npy"), stamps.cpu().numpy())
    world.host_barrier()
    if rank == 0:
        t = np.stack([np.load(os.path.join(world.directory, f"timeline.rank{r}.npy")) for r in range(size)]).reshape(size, rounds, 2)
        t = (t - t[:, 8:, 0].min()) / 100.0                       # us since the first arrival of round 8
        print(f"{size} processes, one barrier launch per rank and round; us on the GPU's wall clock, rounds 8..{rounds - 1}")
        print("round | arrival of each rank's stream after the round's first (rank order) | all ranks left after | round lasted")
        for i in range(8, rounds):
            first = t[:, i, 0].min()
            lags = " ".join(f"{v - first:6.1f}" for v in t[:, i, 0])
            print(f"{i:5d} | {lags} | {t[:, i, 1].max() - first:6.1f} | {t[:, i, 1].max() - t[:, i - 1, 1].max():6.1f}")
        lag = np.sort(t[:, 8:, 0] - t[:, 8:, 0].min(axis=0, keepdims=True), axis=0)     # per round, ranks by arrival
        print("mean arrival after the round's first, k-th to arrive: " + " ".join(f"{v:.1f}" for v in lag.mean(axis=1)))
        own = (t[:, 8:, 1] - t[:, 8:, 0]).mean(axis=1)
        print("mean time between a rank's own two stamps (rank order): " + " ".join(f"{v:.1f}" for v in own), flush=True)
    world.close()
    return 0


def main() -> int:
    if "--timeline" in sys.argv:
        return timeline(ipc.IpcWorld.from_env())
    as_json = "--json" in sys.argv
    sizes = (64, 1024, 4096, 16384, 65536, 262144)
    if "--sizes" in sys.argv:
        sizes = tuple(int(v) for v in sys.argv[sys.argv.index("--sizes") + 1].split(","))
    world = ipc.IpcWorld.from_env()
    rank, size = world.rank, world.world_size
    lib = world.lib

    def timed(fn, reps=16, warm=8, blocks=5):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        world.host_barrier()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(blocks + 1)]
        ev[0].record()
        for b in range(blocks):
            for _ in range(reps):
                fn()
            ev[b + 1].record()
        torch.cuda.synchronize()
        world.check()
        us = sorted(ev[b].elapsed_time(ev[b + 1]) * 1000 / reps for b in range(blocks))
        return us[blocks // 2], us[0]

    def show(pair):
        return "-" if pair is None else f"{pair[0]:.0f} ({pair[1]:.0f})"

    if rank == 0 and not as_json:
        print(f"{size} processes on one GPU; us per collective on rank 0's stream", flush=True)
        print(f"{'per buffer':>10s} {'barrier':>10s} | {'one-shot x3':>11s} {'fused':>11s} | {'rs x3':>10s} {'fused':>10s} | "
              f"{'ag x3':>10s} {'fused':>10s} | {'two-shot x3':>11s} {'fused':>11s} | {'tree x3':>11s} {'fused':>11s}", flush=True)
    for kib in sizes:
        numel = (kib << 9) // (8 * size) * (8 * size)      # whole 16-byte vectors per rank's share in any world
        t = world.empty(numel, torch.bfloat16)
        t.copy_(torch.randn(numel, dtype=torch.bfloat16) * 0.01)
        ptrs = _lib.ptr_array(world._tables[t.data_ptr()][0])
        out = torch.empty_like(t)
        share = torch.empty(numel // size, dtype=torch.bfloat16, device=t.device)
        part = t[: numel // size]                       # all-gather: every rank contributes 1/W of the buffer
        gathered = torch.empty((size, numel // size), dtype=torch.bfloat16, device=t.device)

        def stream():
            return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

        def between_barriers(call):
            def run():
                world.barrier()
                assert call() == 0
                world.barrier()
            return run

        us = [timed(world.barrier)]
        us.append(timed(between_barriers(lambda: lib.tccl_all_reduce_sum(ptrs, size, out.data_ptr(), numel, 0, stream()))))
        us.append(timed(lambda: world.one_shot_all_reduce(t, out=out, fused=True)))
        us.append(timed(between_barriers(lambda: lib.tccl_reduce_scatter_sum(ptrs, size, rank, share.data_ptr(), numel, 0, stream()))))
        us.append(timed(lambda: world.reduce_scatter(t, out=share, fused=True)))
        us.append(timed(between_barriers(lambda: lib.tccl_all_gather(ptrs, size, gathered.data_ptr(), part.numel() * 2, stream()))))
        us.append(timed(lambda: world.all_gather(part, out=gathered, fused=True)))
        us.append(timed(lambda: (t.mul_(1.0 / size), world.two_shot_all_reduce(t, own_barriers=False))))
        us.append(timed(lambda: (t.mul_(1.0 / size), world.two_shot_all_reduce(t))))
        trees = size in (2, 4, 8)
        us.append(timed(lambda: (t.mul_(1.0 / size), world.double_tree_all_reduce(t, own_barriers=False))) if trees else None)
        us.append(timed(lambda: (t.mul_(1.0 / size), world.double_tree_all_reduce(t))) if trees else None)
        if rank == 0 and as_json:
            print(json.dumps({"ipc_forms": True, "processes": size, "kib_per_buffer": kib,
                              "median_us": {c: None if p is None else round(p[0], 1) for c, p in zip(COLUMNS, us)}}), flush=True)
        elif rank == 0:
            label = f"{kib} KiB" if kib < 1024 else f"{kib >> 10} MiB"
            us = [show(p) for p in us]
            print(f"{label:>10s} {us[0]:>10s} | {us[1]:>11s} {us[2]:>11s} | {us[3]:>10s} {us[4]:>10s} | "
                  f"{us[5]:>10s} {us[6]:>10s} | {us[7]:>11s} {us[8]:>11s} | {us[9]:>11s} {us[10]:>11s}", flush=True)
    world.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
