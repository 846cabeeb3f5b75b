"""The reference's all-reduce self-test (triton_one_shot_all_reduce_no_128.py:99-129) as a program
for ``python -m tccl_amd.launch``: rank and world size come from the environment, the buffer is
filled with the rank, and the sum must be W(W-1)/2 everywhere."""
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import tccl_amd                       # noqa: E402
from tccl_amd import ipc              # noqa: E402

if __name__ == "__main__":
    rank = int(os.environ["RANK"])
    world_size = int(os.environ["WORLD_SIZE"])
    world = ipc.IpcWorld.from_env()
    tensor = world.empty(8192, torch.bfloat16).fill_(rank)
    world.barrier()
    output = tccl_amd.one_shot_all_reduce(tensor)
    world.barrier()
    world.check()
    print("OUTPUT", rank, world_size, output[:4].tolist(), flush=True)
    assert output.eq(world_size * (world_size - 1) // 2).all().item()
    world.close()
    sys.exit(int(sys.argv[1]) if len(sys.argv) > 1 and rank == 1 else 0)
