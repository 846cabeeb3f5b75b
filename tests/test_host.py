"""Host-side logic that needs no GPU: the virtual-rank registry and the wrappers'
preconditions (the reference's assertions, raised before anything is launched)."""
import os
import subprocess
import sys

import pytest
import torch

import tccl_amd


def make_group(world=4, numel=64, dtype=torch.bfloat16):
    return tccl_amd.register([torch.zeros(numel, dtype=dtype) for _ in range(world)])


def test_rendezvous_finds_rank_and_peers():
    g = make_group(4)
    for r in range(4):
        h = tccl_amd.rendezvous(g.tensor(r))
        assert h.rank == r and h.world_size == 4
        assert h.buffer_ptrs == tuple(t.data_ptr() for t in g.tensors)
        assert list(h.buffer_ptrs_host) == list(h.buffer_ptrs)
    tccl_amd.unregister(g)


def test_rendezvous_accepts_prefix_views_only():
    g = make_group(2, 128)
    t = g.tensor(1)
    assert tccl_amd.rendezvous(t[:32]).rank == 1            # triton_reduce_scatter.py:222 passes tensor[:size]
    assert tccl_amd.rendezvous(t.view(2, 64)).rank == 1
    with pytest.raises(RuntimeError, match="first element"):
        tccl_amd.rendezvous(t[8:])
    with pytest.raises(RuntimeError, match="contiguous"):
        tccl_amd.rendezvous(t[::2])
    with pytest.raises(RuntimeError, match="registered"):
        tccl_amd.rendezvous(torch.zeros(8))
    tccl_amd.unregister(g)
    with pytest.raises(RuntimeError, match="registered"):
        tccl_amd.rendezvous(t)


def test_group_validation():
    a = torch.zeros(16)
    with pytest.raises(ValueError, match="own allocation"):
        tccl_amd.register([a, a])
    with pytest.raises(ValueError, match="share shape"):
        tccl_amd.register([torch.zeros(16), torch.zeros(8)])
    with pytest.raises(ValueError, match="whole"):
        tccl_amd.register([torch.zeros(16)[4:], torch.zeros(12)])
    with pytest.raises(ValueError):
        tccl_amd.register([])


def test_wrapper_preconditions_match_the_reference():
    """triton_one_shot_all_reduce_no_128.py:73-76, triton_reduce_scatter.py:101-104,
    triton_all_gather.py:73-75, triton_double_tree_allreduce.py:344-347."""
    g = make_group(4, 64, torch.bfloat16)
    t = g.tensor(0)
    with pytest.raises(AssertionError, match="128-bit aligned"):
        tccl_amd.one_shot_all_reduce(t[:10])            # the reference's bound here is 4 elements (:70, :74)
    with pytest.raises(AssertionError, match="128-bit aligned"):
        tccl_amd.one_shot_reduce_scatter(t[:40])        # 40 % (8*4) != 0
    with pytest.raises(AssertionError, match="128-bit aligned"):
        tccl_amd.one_shot_all_gather(t[:12], 4)
    with pytest.raises(AssertionError, match="128-bit aligned"):
        tccl_amd.double_tree_all_reduce(t[:12])
    with pytest.raises(AssertionError, match="world_size"):
        tccl_amd.one_shot_all_gather(t, 8)
    tccl_amd.unregister(g)
    gi = make_group(2, 64, torch.int32)
    with pytest.raises(AssertionError, match="bfloat16"):
        tccl_amd.one_shot_all_reduce(gi.tensor(0))
    with pytest.raises(AssertionError, match="bfloat16"):
        tccl_amd.one_shot_reduce_scatter(gi.tensor(0))
    with pytest.raises(AssertionError, match="bfloat16"):
        tccl_amd.double_tree_all_reduce(gi.tensor(0))
    tccl_amd.unregister(gi)


def test_names():
    assert tccl_amd.reduce_scatter is tccl_amd.one_shot_reduce_scatter
    assert tccl_amd.all_gather is tccl_amd.one_shot_all_gather


def test_launcher_sets_the_environment_and_hands_on_exit_codes(tmp_path):
    """python -m tccl_amd.launch on a program that needs no GPU: every rank sees its RANK, the
    common WORLD_SIZE and rendezvous directory; a failing rank's exit code is the launcher's."""
    prog = tmp_path / "prog.py"
    prog.write_text("import os, sys\n"
                    "r, w, d = os.environ['RANK'], os.environ['WORLD_SIZE'], os.environ['TCCL_RENDEZVOUS_DIR']\n"
                    "assert os.environ['LOCAL_RANK'] == '0' and os.path.isdir(d)\n"
                    "open(os.path.join(sys.argv[1], 'seen' + r), 'w').write(w + ' ' + d)\n"
                    "sys.exit(int(sys.argv[2]) if r == '2' else 0)\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cmd = [sys.executable, "-m", "tccl_amd.launch", "--nproc-per-node", "3", str(prog), str(tmp_path)]
    assert subprocess.run(cmd + ["0"], cwd=root, timeout=60).returncode == 0
    seen = [(tmp_path / f"seen{r}").read_text() for r in range(3)]
    assert all(s.startswith("3 ") for s in seen) and len(set(seen)) == 1
    assert not os.path.exists(seen[0].split(" ", 1)[1]), "the rendezvous directory is removed afterwards"
    assert subprocess.run(cmd + ["5"], cwd=root, timeout=60).returncode == 5
    assert subprocess.run(cmd[:4] + ["9", str(prog)], cwd=root, timeout=60, stderr=subprocess.DEVNULL).returncode == 2


def test_launcher_stops_the_peers_of_a_failed_rank_and_keeps_its_time_limit(tmp_path):
    """A rank that fails leaves peers that would wait for it: they are stopped after the grace period and the
    launcher hands on the failed rank's code; ranks still running at the time limit are stopped with 124."""
    import time
    prog = tmp_path / "prog.py"
    prog.write_text("import os, sys, time\n"
                    "if os.environ['RANK'] == sys.argv[1]:\n"
                    "    sys.exit(7)\n"
                    "time.sleep(120)\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cmd = [sys.executable, "-m", "tccl_amd.launch", "--nproc-per-node", "3"]
    t0 = time.monotonic()
    assert subprocess.run(cmd + ["--grace", "1", str(prog), "1"], cwd=root, timeout=60).returncode == 7
    assert subprocess.run(cmd + ["--timeout", "1", str(prog), "none"], cwd=root, timeout=60).returncode == 124
    assert time.monotonic() - t0 < 30


def test_world_from_environment_needs_a_launcher(monkeypatch):
    from tccl_amd import ipc
    for name in ("RANK", "WORLD_SIZE", "TCCL_RENDEZVOUS_DIR"):
        monkeypatch.delenv(name, raising=False)
    with pytest.raises(RuntimeError, match="tccl_amd.launch"):
        ipc.IpcWorld.from_env()


def test_a_rank_of_a_process_group_never_runs_its_peers_work():
    """A buffer whose peers belong to other processes: everything that would launch every rank's steps
    from this process refuses it (W processes doing that would reduce the mapped buffers W times over)."""
    from tccl_amd import symm
    own = torch.zeros(64, dtype=torch.bfloat16)
    others = [torch.zeros(64, dtype=torch.bfloat16) for _ in range(3)]
    ptrs = [others[0].data_ptr(), own.data_ptr(), others[1].data_ptr(), others[2].data_ptr()]
    group = symm.register_remote(own, 1, ptrs)                       # no IpcWorld behind it
    assert tccl_amd.rendezvous(own).rank == 1 and group.world is None
    with pytest.raises(RuntimeError, match="other processes"):
        tccl_amd.double_tree_all_reduce(own)
    with pytest.raises(RuntimeError, match="other processes"):
        tccl_amd.two_shot_all_reduce(own)
    with pytest.raises(RuntimeError, match="other processes"):
        tccl_amd.all_reduce(own, "double_tree")
    with pytest.raises(RuntimeError, match="other processes"):
        tccl_amd.double_tree_all_reduce_world(group)
    with pytest.raises(RuntimeError, match="other processes"):
        tccl_amd.two_shot_all_reduce_world(group)
    with pytest.raises(RuntimeError, match="other processes"):
        tccl_amd.DoubleTreePlan(group)
    with pytest.raises(ValueError, match="unknown all-reduce algorithm"):
        tccl_amd.all_reduce(own, "ring")
    tccl_amd.unregister(group)


def test_wrappers_hand_a_process_groups_collectives_to_its_world():
    """With the IpcWorld behind the group the reference's names run that world's per-rank forms."""
    from tccl_amd import symm

    class World:
        world_size = 2
        calls = []

        def one_shot_all_reduce(self, t, out=None):
            self.calls.append("one_shot")
            return out

        def reduce_scatter(self, t, out=None):
            self.calls.append("reduce_scatter")
            return out

        def all_gather(self, t, out=None):
            self.calls.append("all_gather")
            return out

        def two_shot_all_reduce(self, t):
            self.calls.append("two_shot")
            return t

        def double_tree_all_reduce(self, t, chunk_elems=0):
            self.calls.append("double_tree")
            return t

        def all_reduce(self, t, algorithm):
            self.calls.append("all_reduce:" + algorithm)
            return t

    own, other = torch.zeros(64, dtype=torch.bfloat16), torch.zeros(64, dtype=torch.bfloat16)
    world = World()
    group = symm.register_remote(own, 0, [own.data_ptr(), other.data_ptr()], world=world)
    assert group.world is world
    tccl_amd.one_shot_all_reduce(own)
    tccl_amd.reduce_scatter(own)
    tccl_amd.all_gather(own, 2)
    tccl_amd.two_shot_all_reduce(own)
    tccl_amd.double_tree_all_reduce(own)
    tccl_amd.all_reduce(own, "auto")
    assert world.calls == ["one_shot", "reduce_scatter", "all_gather", "two_shot", "double_tree", "all_reduce:auto"]
    with pytest.raises(ValueError, match="per-rank"):
        tccl_amd.one_shot_all_reduce(own, cfg=tccl_amd.LaunchCfg())
    with pytest.raises(ValueError, match="per-rank pipelined kernel only"):
        tccl_amd.double_tree_all_reduce(own, fused=True)
    tccl_amd.unregister(group)


def test_ipc_world_refuses_a_directory_another_run_has_used(tmp_path):
    """The handle files have fixed names: a rank that found its own files from an earlier run would go on
    to map allocations that no longer exist.  Refused before anything touches the GPU."""
    from tccl_amd import ipc
    (tmp_path / "pad0.rank1").write_bytes(b"x" * 64)
    with pytest.raises(RuntimeError, match="another run"):
        ipc.IpcWorld(1, 2, str(tmp_path))
    ipc._refuse_used_directory(str(tmp_path), 0)                     # rank 0 has no file there yet: fine
    with pytest.raises(RuntimeError, match="cannot be read"):
        ipc.IpcWorld(0, 2, str(tmp_path / "missing"))


def test_ipc_world_picks_the_all_reduce_by_size_and_world():
    from tccl_amd import ipc

    class Fake(ipc.IpcWorld):
        def __init__(self, world_size):                               # no GPU, no files
            self.world_size, self.rank = world_size, 0

    mib = 1 << 19                                                     # bf16 elements per MiB
    assert Fake(8).auto_algorithm(torch.empty(8 * mib, dtype=torch.bfloat16)) == "one_shot"
    assert Fake(8).auto_algorithm(torch.empty(8 * mib + 64, dtype=torch.bfloat16)) == "two_shot"
    assert Fake(8).auto_algorithm(torch.empty(8 * mib + 8, dtype=torch.bfloat16)) == "one_shot"      # shares would be ragged
    assert Fake(4).auto_algorithm(torch.empty(64 * mib, dtype=torch.bfloat16)) == "one_shot"
    assert Fake(2).auto_algorithm(torch.empty(64 * mib, dtype=torch.bfloat16)) == "one_shot"
    assert Fake(5).auto_algorithm(torch.empty(5 * 16 * mib, dtype=torch.float32)) == "two_shot"
