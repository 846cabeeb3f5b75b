"""What the collectives cost when every rank is a process of its own on the one GPU:

    python -m tccl_amd.launch --nproc-per-node 8 benchlib/ipc_timing.py

Rank 0 prints, per buffer size, the mean time of: the blockwise barrier alone; barrier + every
rank's one-shot all-reduce + barrier; the per-rank two-shot all-reduce and the per-rank
pipelined double tree (each between its two barriers, after a scaling of the buffer that keeps
the values finite).  On one GPU these are dominated by the processes' queues taking turns, not
by the kernels: compare with the one-launch forms in bench.py."""
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import tccl_amd                       # noqa: E402
from tccl_amd import ipc              # noqa: E402


def main() -> int:
    world = ipc.IpcWorld.from_env()
    rank, size = world.rank, world.world_size

    def timed(fn, reps=20, warm=5):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        world.host_barrier()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        world.check()
        return e0.elapsed_time(e1) * 1000 / reps

    for mib in (1, 16, 64):
        numel = mib << 19
        t = world.empty(numel, torch.bfloat16)
        t.copy_(torch.randn(numel, dtype=torch.bfloat16) * 0.01)

        def all_reduce():
            world.barrier()
            tccl_amd.one_shot_all_reduce(t)
            world.barrier()

        us_barrier = timed(world.barrier)
        us_one_shot = timed(all_reduce)
        us_two_shot = timed(lambda: (t.mul_(1.0 / size), world.two_shot_all_reduce(t)))
        line = (f"{mib} MiB per buffer, {size} processes: barrier {us_barrier:.1f} us; barrier + one-shot all-reduce + barrier "
                f"{us_one_shot:.1f} us; two-shot per rank {us_two_shot:.1f} us")
        if size in (2, 4, 8):
            us_tree = timed(lambda: (t.mul_(1.0 / size), world.double_tree_all_reduce(t)))
            line += f"; double tree per rank {us_tree:.1f} us"
        if rank == 0:
            print(line, flush=True)
    world.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
