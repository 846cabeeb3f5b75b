"""One rank of a reference-style per-rank program, run as its own process (started by
test_ipc_gpu.py, W of them on one GPU): allocate a symmetric buffer, fill it with the
reference's recipe, meet the peers in the device-side barrier, run the collectives, leave the
results where the parent can compare them with the oracle.

    python ipc_rank_program.py <rank> <world> <directory> <mode>
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import tccl_amd                       # noqa: E402
from tccl_amd import ipc              # noqa: E402


# (name, elements, dtype): a few chunks with a ragged last one; enough chunks for every workgroup
# slot of the GPU to be in use (8 MiB per buffer); fp32
DOUBLE_TREE_SHAPES = (("small", 98_760, torch.bfloat16), ("big", 4_194_304, torch.bfloat16),
                      ("f32", 1_048_576 + 8, torch.float32))


# (name, elements per rank's share, dtype): less than a tile; many tiles with a ragged last one; fp32
TWO_SHOT_SHAPES = (("small", 8 * 37, torch.bfloat16), ("big", 8 * 65_537, torch.bfloat16), ("f32", 4 * 20_011, torch.float32))


# (name, elements per rank's share, dtype) for the one-shot kernels that carry their barriers themselves:
# less than one tile in all; many tiles with a ragged last one; fp32; enough tiles for every workgroup of a rank
ONE_SHOT_SHAPES = (("small", 8 * 5, torch.bfloat16), ("ragged", 8 * 4099, torch.bfloat16), ("f32", 4 * 10_007, torch.float32),
                   ("big", 8 * 131_072, torch.bfloat16))


# elements per rank's share of the three buffer sizes of the mixed sequence: one workgroup per rank,
# a few dozen, and every workgroup a rank's launch may hold
MIXED_SHARES = (("tiny", 8 * 3), ("mid", 8 * 4099), ("big", 8 * 131_072))
MIXED_ROUNDS = 4


def AUTO_SIZES(world_size, edge):
    """(name, bf16 elements): small; at the threshold of "auto"; one step (W vectors) above it; a buffer
    large enough that a one-shot all-reduce is three launches again."""
    return (("small", 8 * world_size * 33), ("at", edge), ("above", edge + 8 * world_size), ("large", 4 * edge))


def fill(t, numel, dtype, seed):
    torch.manual_seed(seed)
    if dtype == torch.bfloat16:
        t.copy_(torch.randn(numel, dtype=dtype))
    else:
        t.copy_(torch.rand(numel, dtype=dtype) * 2 - 1)


def save(directory, name, rank, t):
    t = t.detach().cpu().contiguous()
    view = {2: torch.int16, 4: torch.int32, 1: torch.int8}[t.element_size()]
    np.save(os.path.join(directory, f"{name}.rank{rank}.npy"), t.view(view).numpy())


def main():
    rank, world_size, directory, mode = int(sys.argv[1]), int(sys.argv[2]), sys.argv[3], sys.argv[4]
    world = ipc.IpcWorld(rank, world_size, directory)
    print(f"rank {rank}: pads exchanged", flush=True)
    if mode == "missing_peer":
        # rank 0 waits in the barrier, nobody else comes: its wait must expire and be reported;
        # after a collective reset of the pads the barrier works again for everybody
        reported = False
        if rank == 0:
            world.barrier(spin_limit=2000)
            try:
                world.check()
            except tccl_amd.TcclError as e:
                print(f"rank 0: reported: {e}", flush=True)
                reported = True
        world.reset()
        for _ in range(3):
            world.barrier()
        world.check()
        print(f"rank {rank}: barrier works after the reset", flush=True)
        world.close()
        return 42 if reported else (0 if rank != 0 else 1)

    if mode == "one_shot_rank":
        # all-reduce, reduce-scatter and all-gather as ONE launch per rank each, the leading and the
        # trailing barrier inside the kernel: no barrier launch anywhere, no host barrier between the
        # rounds -- a rank refills its buffer as soon as its own kernels are done, which is exactly
        # what the trailing barrier has to make safe
        for tag, per_rank, dtype in ONE_SHOT_SHAPES:
            numel = per_rank * world_size
            t = world.empty(numel, dtype)
            for round_ in range(2):
                fill(t, numel, dtype, 100 * round_ + rank)
                if (round_ + rank) % 3 == 0:
                    torch.cuda._sleep(2_000_000)          # ranks out of step
                if round_ == 0:
                    outs = (world.one_shot_all_reduce(t), world.reduce_scatter(t), world.all_gather(t))
                else:                                      # the reference's names find the world by themselves
                    outs = (tccl_amd.one_shot_all_reduce(t), tccl_amd.reduce_scatter(t), tccl_amd.all_gather(t, world_size))
                for name, o in zip(("all_reduce", "reduce_scatter", "all_gather"), outs):
                    save(directory, f"rank_{name}_{tag}.{round_}", rank, o)
            world.check()
            print(f"rank {rank}: one-shot kernels {tag} done", flush=True)
        pad = world._kernel_pads(world.ONE_SHOT_PAD_BYTES, "one_shot")
        own = ipc._as_tensor(pad[rank], world.ONE_SHOT_PAD_BYTES, world.device).view(torch.int32)
        world.barrier()
        left = int(own.ne(0).sum())
        world.check()
        world.close()
        if left:
            print(f"rank {rank}: {left} words of the signal pad are not zero after the collectives", flush=True)
            return 5
        return 0

    if mode == "mixed_sequence":
        # collectives of different kinds and very different sizes back to back, ranks out of step, no
        # meeting on the host anywhere: a launch with many workgroups follows one with few on the same
        # pads (and the other way round), one-shot, two-shot and double-tree kernels follow each other.
        # Every kernel's flags must land where its peers' kernels of the SAME call look for them and
        # nowhere else, whatever ran just before.
        bufs = {tag: world.empty(share * world_size, torch.bfloat16) for tag, share in MIXED_SHARES}
        inplace = {tag: world.empty(share * world_size, torch.bfloat16) for tag, share in MIXED_SHARES}
        keep = {}
        for tag, share in MIXED_SHARES:
            fill(bufs[tag], share * world_size, torch.bfloat16, 700 + rank)
            keep[tag] = bufs[tag].clone()
        trees = world_size in (2, 4, 8)
        results = []
        for round_ in range(MIXED_ROUNDS):
            if (round_ + rank) % 3 == 0:
                torch.cuda._sleep(3_000_000)
            order = ("tiny", "big", "mid", "big", "tiny") if round_ % 2 == 0 else ("big", "tiny", "mid", "tiny", "big")
            for step, tag in enumerate(order):
                kind = ("reduce_scatter", "all_reduce", "all_gather", "two_shot", "double_tree")[(step + round_) % 5]
                if kind == "double_tree" and not trees:
                    kind = "two_shot"
                if kind == "reduce_scatter":
                    out = world.reduce_scatter(bufs[tag], fused=True)
                elif kind == "all_reduce":
                    out = world.one_shot_all_reduce(bufs[tag], fused=True)
                elif kind == "all_gather":
                    out = world.all_gather(bufs[tag], fused=True)
                else:                                                  # in place: refill first (the last call's trailing
                    inplace[tag].copy_(keep[tag])                      # barrier has made that safe)
                    out = (world.two_shot_all_reduce(inplace[tag]) if kind == "two_shot"
                           else world.double_tree_all_reduce(inplace[tag]))
                results.append((f"mixed_{round_}_{step}_{kind}_{tag}", out))
        torch.cuda.synchronize()
        world.check()
        for name, out in results:
            save(directory, name, rank, out)
        if rank == 0:
            print("SEQUENCE " + " ".join(name for name, _ in results), flush=True)
        world.close()
        return 0

    if mode == "one_shot_missing_peer":
        # rank 0 starts an all-reduce with a small spin limit and nobody joins: its kernel must end by
        # itself and the rank must be told; after a collective reset everybody's collectives work
        numel = 8 * world_size * 1031
        t = world.empty(numel, torch.bfloat16)
        reported = False
        if rank == 0:
            cfg = tccl_amd._lib.PipelineCfg()
            cfg.spin_limit = 2000
            world.one_shot_all_reduce(t, cfg=cfg)
            try:
                world.check()
            except tccl_amd.TcclError as e:
                print(f"rank 0: reported: {e}", flush=True)
                reported = True
        world.reset()
        for round_ in range(2):
            fill(t, numel, torch.bfloat16, 100 * round_ + rank)
            save(directory, f"after_reset.{round_}", rank, world.one_shot_all_reduce(t))
        world.check()
        world.close()
        return 42 if reported else (0 if rank != 0 else 1)

    if mode == "kernel_timeout_reset":
        # a wait INSIDE a collective's kernel expires on some ranks (rank 1's stream is held back behind
        # the leading barrier while the others run the two-shot kernel with a small spin limit); the
        # flags they leave standing in the kernel pads must be gone after reset(), or the next
        # collective on the same pads would pass its barrier early and return partial sums
        numel = 8 * world_size * 2053
        t = world.empty(numel, torch.bfloat16)
        fill(t, numel, torch.bfloat16, rank)
        cfg = tccl_amd._lib.PipelineCfg()
        cfg.spin_limit = 3000 if rank != 1 else 0
        # (the pads first: allocating them is a meeting of the ranks on the host and waits for the own stream)
        pads = world._kernel_pads(world.TWO_SHOT_PAD_BYTES, "two_shot")
        world.barrier()
        if rank == 1:
            torch.cuda._sleep(400_000_000)                # about 0.2 s on the GPU, bounded
        ptrs = tccl_amd._lib.ptr_array(world._tables[t.data_ptr()][0])
        cfg.timeout_flag = world._flag
        import ctypes
        rc = world.lib.tccl_two_shot_all_reduce_rank(ptrs, None, pads, world.TWO_SHOT_PAD_BYTES, world_size, rank, numel, 0,
                                                     ctypes.byref(cfg), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, rc
        reported = False
        try:
            world.check()
        except tccl_amd.TcclError as e:
            print(f"rank {rank}: reported: {e}", flush=True)
            reported = True
        world.host_barrier()                              # every rank has looked at its own flag
        try:
            world.check()                                 # ... and now also sees what the peers published
        except tccl_amd.TcclError as e:
            print(f"rank {rank}: told: {e}", flush=True)
            reported = True
        world.reset()
        for round_ in range(2):
            fill(t, numel, torch.bfloat16, 100 * (round_ + 1) + rank)
            out = world.two_shot_all_reduce(t)
            world.check()
            save(directory, f"after_kernel_timeout.{round_}", rank, out)
            world.host_barrier()
        world.close()
        return 42 if reported else 1

    if mode == "auto":
        # IpcWorld.all_reduce: every algorithm by name and "auto" at one size either side of its threshold
        # (and one size above the point where a one-shot collective stops being one launch)
        edge = world.ONE_SHOT_MAX_BYTES // 2                     # bf16 elements at the threshold
        for tag, numel in AUTO_SIZES(world_size, edge):
            t = world.empty(numel, torch.bfloat16)
            for algorithm in ("auto", "one_shot", "two_shot", "double_tree"):
                fill(t, numel, torch.bfloat16, rank)              # the in-place forms overwrite the buffer
                picked = world.auto_algorithm(t) if algorithm == "auto" else algorithm
                via_wrapper = algorithm in ("auto", "two_shot")   # the reference-side names lead to the same place
                out = tccl_amd.all_reduce(t, algorithm) if via_wrapper else world.all_reduce(t, algorithm)
                world.check()
                save(directory, f"auto_{tag}.{algorithm}", rank, out)
                if rank == 0:
                    print(f"PICKED {tag} {algorithm} {picked}", flush=True)
                world.host_barrier()                              # nobody refills before everybody has saved
        world.close()
        return 0

    if mode == "reference_mains":
        # the self-tests at the bottom of the reference's four kernel files, with a process per rank
        # as there: triton_one_shot_all_reduce_no_128.py:116-127, triton_reduce_scatter.py:185-211,
        # triton_all_gather.py:117-133, triton_double_tree_allreduce.py:388-410
        total = world_size * (world_size - 1) // 2
        tensor = world.empty(8192, torch.bfloat16).fill_(rank)
        world.barrier()
        output = tccl_amd.one_shot_all_reduce(tensor)
        assert output.eq(total).all().item(), "all-reduce"
        share = tccl_amd.reduce_scatter(tensor)
        assert share.shape == (8192 // world_size,) and share.eq(total).all().item(), "reduce-scatter"
        gathered = tccl_amd.all_gather(tensor, world_size)
        want = torch.arange(world_size, dtype=torch.bfloat16, device=tensor.device).unsqueeze(1).expand(world_size, 8192)
        assert gathered.shape == (world_size, 8192) and gathered.eq(want).all().item(), "all-gather"
        world.barrier()
        if world_size in (2, 4, 8):
            output = world.double_tree_all_reduce(tensor)
            assert output.eq(total).all().item() and tensor.eq(total).all().item(), "double tree"
        world.check()
        print(f"rank {rank}: OUTPUT {world_size} {output[:4].tolist()}", flush=True)
        world.close()
        return 0

    if mode == "graph":
        # [barrier, all-reduce, barrier] recorded once into a HIP graph by every rank and replayed with
        # new inputs: the barrier needs no host-side state (its pads reset themselves), which is what
        # the reference means by graph-friendly (triton_barrier.py:47-54)
        numel = 8 * 3001
        tensor = world.empty(numel, torch.bfloat16)
        out = torch.empty(numel, dtype=torch.bfloat16, device=tensor.device)

        def enqueue():
            world.barrier()
            tccl_amd.one_shot_all_reduce(tensor, out=out)
            world.barrier()

        tensor.fill_(rank)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            enqueue()                                  # warm-up outside the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        world.host_barrier()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            enqueue()
        for rep in range(4):
            torch.manual_seed(100 * rep + rank)
            tensor.copy_(torch.randn(numel, dtype=torch.bfloat16))
            out.zero_()
            graph.replay()
            world.check()
            save(directory, f"graph.{rep}", rank, out)
            world.host_barrier()                       # nobody refills before everybody has saved
        print(f"rank {rank}: graph replayed 4 times", flush=True)
        world.close()
        return 0

    if mode == "barrier_test":
        # the reference's own barrier test (triton_barrier.py:155-190): 32 blocks per rank, one
        # launch per rank, then look at the pad -- which must be all zero again
        for _ in range(3):
            world.barrier(blocks=32)
        world.check()
        pad = world.signal_pad().cpu()
        world.close()
        if int(pad.ne(0).sum()) != 0:
            print(f"rank {rank}: pad not zero after the barrier: {pad.nonzero().flatten().tolist()[:8]}", flush=True)
            return 4
        print(f"rank {rank}: barrier test passed, pad is zero", flush=True)
        return 0

    if mode == "barrier_storm":
        # Barriers back to back with nothing but a tiny kernel between them, ranks arriving out of
        # step: before barrier i every rank writes i into its cell, after it every rank reads all
        # cells, and a second barrier keeps anybody from writing i + 1 before all have read i.
        rounds = 120
        cell = world.empty(4, torch.int32)
        cells = world.peers(cell)
        log = torch.zeros((rounds, world_size), dtype=torch.int32, device=cell.device)
        for i in range(rounds):
            if (i + rank) % 5 == 0:
                torch.cuda._sleep(300_000 * (1 + rank % 3))
            cell.fill_(i + 1)
            world.barrier()
            log[i] = torch.stack([c[0] for c in cells])
            world.barrier()
        world.check()
        want = torch.arange(1, rounds + 1, dtype=torch.int32).unsqueeze(1).expand(rounds, world_size)
        got = log.cpu()
        world.close()
        if not torch.equal(got, want):
            bad = (got != want).nonzero()[0].tolist()
            print(f"rank {rank}: round {bad[0]} read {got[bad[0]].tolist()}", flush=True)
            return 3
        print(f"rank {rank}: {2 * rounds} barriers in a row, every read in step", flush=True)
        return 0

    if mode == "double_tree":
        # one launch per rank of the pipelined double tree, ranks signalling each other through
        # pads in each other's memory; two rounds per shape on the same buffers and pads
        for tag, numel, dtype in DOUBLE_TREE_SHAPES:
            t = world.empty(numel, dtype)
            for round_ in range(2):
                torch.manual_seed(100 * round_ + rank)
                if dtype == torch.bfloat16:
                    t.copy_(torch.randn(numel, dtype=dtype))
                else:
                    t.copy_(torch.rand(numel, dtype=dtype) * 2 - 1)
                # first pass: one launch per rank, the kernel's own barriers; second pass: a barrier launch either side
                out = world.double_tree_all_reduce(t, own_barriers=(round_ == 0))
                world.check()
                save(directory, f"double_tree_{tag}.{round_}.out", rank, out)
                save(directory, f"double_tree_{tag}.{round_}.buf", rank, t)
                world.host_barrier()          # nobody refills before everybody has saved
            print(f"rank {rank}: double tree {tag} done", flush=True)
        world.close()
        return 0

    if mode == "two_shot":
        # one launch per rank of the two-shot kernel: the blockwise barrier between its shots is a
        # barrier between kernels of different owners
        for tag, numel, dtype in TWO_SHOT_SHAPES:
            numel *= world_size
            t = world.empty(numel, dtype)
            for round_ in range(2):
                torch.manual_seed(100 * round_ + rank)
                if dtype == torch.bfloat16:
                    t.copy_(torch.randn(numel, dtype=dtype))
                else:
                    t.copy_(torch.rand(numel, dtype=dtype) * 2 - 1)
                # first pass: one launch per rank, the kernel's own barriers; second pass: a barrier launch either side
                out = world.two_shot_all_reduce(t, own_barriers=(round_ == 0))
                world.check()
                save(directory, f"two_shot_{tag}.{round_}.out", rank, out)
                save(directory, f"two_shot_{tag}.{round_}.buf", rank, t)
                world.host_barrier()
            print(f"rank {rank}: two-shot {tag} done", flush=True)
        world.close()
        return 0

    numel = 8 * world_size * 4099
    bf = world.empty(numel, torch.bfloat16)
    fp = world.empty(numel // 2, torch.float32)
    for round_ in range(2):
        torch.manual_seed(100 * round_ + rank)
        bf.copy_(torch.randn(numel, dtype=torch.bfloat16))
        torch.manual_seed(100 * round_ + rank)
        fp.copy_(torch.rand(numel // 2, dtype=torch.float32) * 2 - 1)
        world.barrier()                                  # leading barrier: every rank's buffers are filled
        save(directory, f"all_reduce_bf16.{round_}", rank, tccl_amd.one_shot_all_reduce(bf))
        save(directory, f"reduce_scatter_bf16.{round_}", rank, tccl_amd.reduce_scatter(bf))
        save(directory, f"all_gather_bf16.{round_}", rank, tccl_amd.all_gather(bf, world_size))
        save(directory, f"all_reduce_f32.{round_}", rank, tccl_amd.one_shot_all_reduce(fp))
        save(directory, f"reduce_scatter_f32.{round_}", rank, tccl_amd.reduce_scatter(fp))
        world.barrier()                                  # trailing barrier: every rank has read them
        world.check()
        print(f"rank {rank}: round {round_} done", flush=True)
    world.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
