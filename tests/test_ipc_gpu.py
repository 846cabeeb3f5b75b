"""Symmetric buffers owned by separate processes on one GPU: W child processes each allocate their
buffer, exchange IPC handles, meet in the device-side blockwise barrier (one launch per rank, as
the reference's kernels do: triton_barrier.py:39-142) and run the collectives on the mapped
addresses; the parent compares what every rank got with the oracle, bit for bit."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import seeded_randn, seeded_uniform
from oracle import torch_ref

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAM = os.path.join(ROOT, "tests", "ipc_rank_program.py")


def run_ranks(world, directory, mode, timeout=110):
    procs = [subprocess.Popen([sys.executable, PROGRAM, str(r), str(world), str(directory), mode],
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True) for r in range(world)]
    outs, codes = [], []
    try:
        for p in procs:
            out, _ = p.communicate(timeout=timeout)
            outs.append(out)
            codes.append(p.returncode)
    finally:
        for p in procs:                      # exactly the processes started here
            if p.poll() is None:
                p.kill()
                p.wait()
    return codes, outs


def load(directory, name, rank, dtype):
    a = np.load(os.path.join(directory, f"{name}.rank{rank}.npy"))
    return torch.from_numpy(a).view(dtype)


@pytest.mark.parametrize("world", [4, 8])
def test_collectives_across_processes(world, tmp_path):
    assert torch.cuda.is_available()
    print(f"ipc: {world} processes", flush=True)
    codes, outs = run_ranks(world, tmp_path, "collectives")
    assert codes == [0] * world, "\n".join(outs)
    numel = 8 * world * 4099
    per = numel // world
    for round_ in range(2):
        bf = seeded_randn(world, numel, seed_base=100 * round_)
        fp = seeded_uniform(world, numel // 2, seed_base=100 * round_)
        want_bf, want_fp = torch_ref.all_reduce(bf), torch_ref.all_reduce(fp)
        stacked = torch.stack(bf)
        perf = (numel // 2) // world
        for r in range(world):
            assert torch.equal(load(tmp_path, f"all_reduce_bf16.{round_}", r, torch.bfloat16).view(torch.int16),
                               want_bf.view(torch.int16)), f"round {round_} rank {r}: all-reduce bf16"
            assert torch.equal(load(tmp_path, f"reduce_scatter_bf16.{round_}", r, torch.bfloat16).view(torch.int16),
                               want_bf[r * per:(r + 1) * per].view(torch.int16)), f"round {round_} rank {r}: reduce-scatter bf16"
            assert torch.equal(load(tmp_path, f"all_gather_bf16.{round_}", r, torch.bfloat16).view(torch.int16),
                               stacked.view(torch.int16)), f"round {round_} rank {r}: all-gather"
            assert torch.equal(load(tmp_path, f"all_reduce_f32.{round_}", r, torch.float32).view(torch.int32),
                               want_fp.view(torch.int32)), f"round {round_} rank {r}: all-reduce f32"
            assert torch.equal(load(tmp_path, f"reduce_scatter_f32.{round_}", r, torch.float32).view(torch.int32),
                               want_fp[r * perf:(r + 1) * perf].view(torch.int32)), f"round {round_} rank {r}: reduce-scatter f32"


@pytest.mark.parametrize("world", [4, 8])
def test_double_tree_one_launch_per_rank(world, tmp_path):
    """The reference's double-tree design as it runs it: every rank (a process) launches its own
    kernel, and the kernels hand chunks to each other through wait/send on pads in each other's
    memory (triton_double_tree_allreduce.py:175-225, :338-370).  Outputs and the buffers (the
    collective works in place) against the oracle, bit for bit, two rounds per shape."""
    from ipc_rank_program import DOUBLE_TREE_SHAPES
    print(f"ipc: double tree, {world} processes", flush=True)
    codes, outs = run_ranks(world, tmp_path, "double_tree", timeout=150)
    assert codes == [0] * world, "\n".join(outs)
    for tag, numel, dtype in DOUBLE_TREE_SHAPES:
        bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
        for round_ in range(2):
            bufs = (seeded_randn(world, numel, seed_base=100 * round_) if dtype == torch.bfloat16
                    else seeded_uniform(world, numel, seed_base=100 * round_))
            want = torch_ref.double_tree_all_reduce(bufs)[0].view(bits)
            for r in range(world):
                for what in ("out", "buf"):
                    got = load(tmp_path, f"double_tree_{tag}.{round_}.{what}", r, dtype).view(bits)
                    assert torch.equal(got, want), f"{tag} round {round_} rank {r} {what}"


@pytest.mark.parametrize("world", [3, 8])
def test_two_shot_one_launch_per_rank(world, tmp_path):
    """Two-shot all-reduce with every rank (a process) launching its own kernel: the blockwise
    barrier between the shots is then the reference's construct, a barrier between kernels of
    different owners inside the kernel (triton_barrier.py:39-142).  Outputs and buffers against
    the oracle's all-reduce, bit for bit, two rounds per shape."""
    from ipc_rank_program import TWO_SHOT_SHAPES
    print(f"ipc: two-shot, {world} processes", flush=True)
    codes, outs = run_ranks(world, tmp_path, "two_shot", timeout=150)
    assert codes == [0] * world, "\n".join(outs)
    for tag, per_rank, dtype in TWO_SHOT_SHAPES:
        numel = per_rank * world
        bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
        for round_ in range(2):
            bufs = (seeded_randn(world, numel, seed_base=100 * round_) if dtype == torch.bfloat16
                    else seeded_uniform(world, numel, seed_base=100 * round_))
            want = torch_ref.all_reduce(bufs).view(bits)
            for r in range(world):
                for what in ("out", "buf"):
                    got = load(tmp_path, f"two_shot_{tag}.{round_}.{what}", r, dtype).view(bits)
                    assert torch.equal(got, want), f"{tag} round {round_} rank {r} {what}"


@pytest.mark.parametrize("world", [3, 4, 8])
def test_one_shot_kernels_with_their_barriers_inside(world, tmp_path):
    """The reference's form for process-owned ranks (triton_one_shot_all_reduce_no_128.py:46,
    triton_all_gather.py:43): every rank's all-reduce, reduce-scatter and all-gather is ONE launch that
    begins with the blockwise barrier and -- beyond the reference -- ends with one.  bf16 and fp32, two
    rounds per shape with a refill between them and no other synchronisation; against the oracle, bit for bit."""
    from ipc_rank_program import ONE_SHOT_SHAPES
    print(f"ipc: one-shot kernels with barriers inside, {world} processes", flush=True)
    codes, outs = run_ranks(world, tmp_path, "one_shot_rank", timeout=150)
    assert codes == [0] * world, "\n".join(outs)
    for tag, per_rank, dtype in ONE_SHOT_SHAPES:
        numel = per_rank * world
        bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
        for round_ in range(2):
            bufs = (seeded_randn(world, numel, seed_base=100 * round_) if dtype == torch.bfloat16
                    else seeded_uniform(world, numel, seed_base=100 * round_))
            want = torch_ref.all_reduce(bufs).view(bits)
            stacked = torch.stack(bufs).view(bits)
            for r in range(world):
                got = load(tmp_path, f"rank_all_reduce_{tag}.{round_}", r, dtype).view(bits)
                assert torch.equal(got, want), f"{tag} round {round_} rank {r}: all-reduce"
                got = load(tmp_path, f"rank_reduce_scatter_{tag}.{round_}", r, dtype).view(bits)
                assert torch.equal(got, want[r * per_rank:(r + 1) * per_rank]), f"{tag} round {round_} rank {r}: reduce-scatter"
                got = load(tmp_path, f"rank_all_gather_{tag}.{round_}", r, dtype).view(bits)
                assert torch.equal(got, stacked), f"{tag} round {round_} rank {r}: all-gather"


@pytest.mark.parametrize("world", [8, 3, 2, 1])
def test_mixed_sequence_of_kinds_and_sizes_without_host_meetings(world, tmp_path):
    """One-shot, two-shot and double-tree kernels of one workgroup per rank up to every workgroup a rank
    may hold, back to back on the same pads with the ranks out of step and no host meeting: a call with
    many workgroups right after one with few (whose trailing flags a slow peer may not have taken yet)
    and kernels of different families after each other.  Every output against the oracle, bit for bit."""
    from ipc_rank_program import MIXED_SHARES
    print(f"ipc: mixed sequence, {world} processes", flush=True)
    codes, outs = run_ranks(world, tmp_path, "mixed_sequence", timeout=150)
    assert codes == [0] * world, "\n".join(outs)
    names = [line for line in outs[0].splitlines() if line.startswith("SEQUENCE ")][0].split()[1:]
    assert len(names) == 20 and {n.rsplit("_", 1)[1] for n in names} == {"tiny", "mid", "big"}
    want, stacked, tree = {}, {}, {}
    for tag, share in MIXED_SHARES:
        bufs = seeded_randn(world, share * world, seed_base=700)
        want[tag] = torch_ref.all_reduce(bufs).view(torch.int16)
        stacked[tag] = torch.stack(bufs).view(torch.int16)
        if world in (2, 4, 8):                  # the trees add in their own order
            tree[tag] = torch_ref.double_tree_all_reduce(bufs)[0].view(torch.int16)
    shares = dict(MIXED_SHARES)
    for name in names:
        kind, tag = name.split("_", 3)[3].rsplit("_", 1)
        for r in range(world):
            got = load(tmp_path, name, r, torch.bfloat16).view(torch.int16)
            if kind == "reduce_scatter":
                expect = want[tag][r * shares[tag]:(r + 1) * shares[tag]]
            elif kind == "all_gather":
                expect = stacked[tag]
            elif kind == "double_tree":
                expect = tree[tag]
            else:
                expect = want[tag]
            assert torch.equal(got.reshape(expect.shape), expect), f"{name} rank {r}"


def test_one_shot_kernel_with_a_missing_peer_gives_up_and_says_so(tmp_path):
    """Failure handling forced from the host: rank 0 launches its all-reduce with a small spin limit and
    no peer ever does.  The kernel ends by itself at its leading barrier, the rank is told, and after a
    collective reset (which clears the flags it left in the peers' pads) the collective works."""
    world, numel = 2, 8 * 2 * 1031
    codes, outs = run_ranks(world, tmp_path, "one_shot_missing_peer", timeout=90)
    assert codes == [42, 0], "\n".join(outs)
    assert "expired" in outs[0]
    for round_ in range(2):
        want = torch_ref.all_reduce(seeded_randn(world, numel, seed_base=100 * round_)).view(torch.int16)
        for r in range(world):
            assert torch.equal(load(tmp_path, f"after_reset.{round_}", r, torch.bfloat16).view(torch.int16), want)


def test_reset_clears_the_pads_of_the_signalling_kernels(tmp_path):
    """A wait inside the two-shot kernel expires on three of four ranks (forced from the host: the fourth
    rank's stream is held back, the others poll a few thousand times).  They report it, the fourth is told
    through the rendezvous directory, reset() clears every pad -- the kernels' as well as the barrier's --
    and the next collectives on the same pads match the oracle."""
    world, numel = 4, 8 * 4 * 2053
    codes, outs = run_ranks(world, tmp_path, "kernel_timeout_reset", timeout=120)
    assert codes == [42] * world, "\n".join(outs)
    assert sum("reported:" in o for o in outs) >= 1
    for round_ in range(2):
        want = torch_ref.all_reduce(seeded_randn(world, numel, seed_base=100 * (round_ + 1))).view(torch.int16)
        for r in range(world):
            got = load(tmp_path, f"after_kernel_timeout.{round_}", r, torch.bfloat16).view(torch.int16)
            assert torch.equal(got, want), f"round {round_} rank {r}"


def test_all_reduce_by_name_and_auto_either_side_of_the_threshold(tmp_path):
    """IpcWorld.all_reduce with 8 processes: "auto" takes the one-shot kernel up to ONE_SHOT_MAX_BYTES per buffer
    and the two-shot kernel one step above it; every algorithm by name at every size.  One-shot and two-shot
    against the oracle's all-reduce, the double tree against the oracle's double tree, bit for bit."""
    from ipc_rank_program import AUTO_SIZES
    from tccl_amd import ipc
    world = 8
    codes, outs = run_ranks(world, tmp_path, "auto", timeout=160)
    assert codes == [0] * world, "\n".join(outs)
    picked = dict((tuple(line.split()[1:3]), line.split()[3]) for line in outs[0].splitlines() if line.startswith("PICKED"))
    assert picked[("small", "auto")] == "one_shot" and picked[("at", "auto")] == "one_shot"
    assert picked[("above", "auto")] == "two_shot" and picked[("large", "auto")] == "two_shot"
    for tag, numel in AUTO_SIZES(world, ipc.IpcWorld.ONE_SHOT_MAX_BYTES // 2):
        bufs = seeded_randn(world, numel)
        flat = torch_ref.all_reduce(bufs).view(torch.int16)
        tree = torch_ref.double_tree_all_reduce(bufs)[0].view(torch.int16)
        for algorithm in ("auto", "one_shot", "two_shot", "double_tree"):
            want = tree if algorithm == "double_tree" else flat
            for r in range(world):
                got = load(tmp_path, f"auto_{tag}.{algorithm}", r, torch.bfloat16).view(torch.int16)
                assert torch.equal(got, want), f"{tag} {algorithm} rank {r}"


@pytest.mark.parametrize("world", [8, 4])
def test_reference_self_tests_with_a_process_per_rank(world, tmp_path):
    """The `__main__` self-tests of the reference's kernel files (every rank fills its buffer
    with its rank, the sum must be W(W-1)/2 everywhere), run the way the reference runs them:
    one process per rank."""
    codes, outs = run_ranks(world, tmp_path, "reference_mains")
    assert codes == [0] * world, "\n".join(outs)


def test_launcher_runs_a_program_once_per_rank():
    """python -m tccl_amd.launch: RANK / WORLD_SIZE / TCCL_RENDEZVOUS_DIR in the environment of
    every rank, the exit code of a failing rank handed on."""
    cmd = [sys.executable, "-m", "tccl_amd.launch", "--nproc-per-node", "8", os.path.join(ROOT, "tests", "ipc_env_program.py")]
    done = subprocess.run(cmd, cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=150)
    assert done.returncode == 0, done.stdout
    assert done.stdout.count("OUTPUT") == 8 and "[28.0, 28.0, 28.0, 28.0]" in done.stdout
    done = subprocess.run(cmd + ["7"], cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=150)
    assert done.returncode == 7, done.stdout


def test_barrier_and_collective_replayed_from_a_graph_in_every_process(tmp_path):
    """The barrier is graph-friendly in the reference's sense (triton_barrier.py:47-54): every rank
    records [barrier, all-reduce, barrier] into a HIP graph once and replays it four times with new
    inputs; each replay against the oracle."""
    world, numel = 8, 8 * 3001
    codes, outs = run_ranks(world, tmp_path, "graph")
    assert codes == [0] * world, "\n".join(outs)
    for rep in range(4):
        want = torch_ref.all_reduce(seeded_randn(world, numel, seed_base=100 * rep)).view(torch.int16)
        for r in range(world):
            assert torch.equal(load(tmp_path, f"graph.{rep}", r, torch.bfloat16).view(torch.int16), want), f"replay {rep} rank {r}"


def test_reference_barrier_test(tmp_path):
    """triton_barrier.py:155-190 as a per-rank program: 8 ranks, 32 blocks each, one launch per
    rank; afterwards every rank's signal pad is all zero."""
    codes, outs = run_ranks(8, tmp_path, "barrier_test")
    assert codes == [0] * 8, "\n".join(outs)


@pytest.mark.parametrize("world", [3, 8])
def test_barriers_back_to_back_with_ranks_out_of_step(world, tmp_path):
    """A rank may enter its next barrier while a peer has seen, but not yet lowered, the flag of the
    previous one: the sender has to wait for the slot to be lowered, or its new flag is wiped out
    with the old one.  240 barriers per rank with nothing but a tiny kernel between them, some
    ranks delayed now and then; every read between two barriers must see that round's values."""
    print(f"ipc: barriers back to back, {world} processes", flush=True)
    codes, outs = run_ranks(world, tmp_path, "barrier_storm", timeout=150)
    assert codes == [0] * world, "\n".join(outs)


def test_barrier_with_a_missing_peer_gives_up_and_says_so(tmp_path):
    """Failure handling forced from the host: rank 0 enters the barrier with a small spin limit and
    no peer ever does.  Its kernel must end by itself and the rank must be told; the flag it left
    standing in the peer's pad is cleared by a collective reset, after which barriers work again."""
    codes, outs = run_ranks(2, tmp_path, "missing_peer", timeout=90)
    assert codes == [42, 0], "\n".join(outs)
    assert "did not reach the barrier" in outs[0]
    assert all("barrier works after the reset" in o for o in outs)
