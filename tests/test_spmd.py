"""The per-rank program runner: W threads, symmetric allocation by call order, collective
rendezvous, error propagation.  CPU only (the collectives themselves are not launched)."""
import threading

import pytest
import torch

import tccl_amd
from tccl_amd import spmd


def test_allocations_form_groups_in_call_order():
    seen = {}

    def main(rank, world_size):
        a = spmd.empty_strided_p2p((64,), (1,), torch.bfloat16, "cpu", "world").fill_(rank)
        b = spmd.empty_strided_p2p(32, None, torch.float32, "cpu")
        assert spmd.current_rank() == rank and spmd.current_world_size() == world_size
        spmd.rendezvous_barrier()                      # every rank has allocated by now
        ha, hb = tccl_amd.rendezvous(a), tccl_amd.rendezvous(b)
        seen[rank] = (ha.rank, ha.world_size, hb.rank, ha.group is not hb.group, ha.buffer_ptrs)
        return float(a[0])

    assert spmd.run(4, main) == [0.0, 1.0, 2.0, 3.0]
    tables = {v[4] for v in seen.values()}
    assert len(tables) == 1                            # every rank sees the same pointer table
    for rank, (ra, world, rb, distinct, _) in seen.items():
        assert (ra, world, rb, distinct) == (rank, 4, rank, True)
    assert spmd.current_rank() is None


def test_collective_bracket_is_two_barriers():
    order = []
    lock = threading.Lock()

    def main(rank, world_size):
        with lock:
            order.append(("before", rank))
        with spmd.collective() as turn:
            with lock:
                order.append(("inside", rank, turn.first))
        with lock:
            order.append(("after", rank))

    spmd.run(3, main)
    kinds = [o[0] for o in order]
    assert kinds[:3] == ["before"] * 3 and kinds[3:6] == ["inside"] * 3 and kinds[6:] == ["after"] * 3
    assert sum(1 for o in order if o[0] == "inside" and o[2]) == 1      # exactly one rank goes first


def test_a_failing_rank_releases_the_others():
    def main(rank, world_size):
        if rank == 2:
            raise ValueError("rank 2 gives up")
        with spmd.collective():
            pass

    with pytest.raises(ValueError, match="rank 2 gives up"):
        spmd.run(4, main)


def test_precondition_failure_inside_a_collective_propagates():
    def main(rank, world_size):
        t = spmd.empty_strided_p2p((10,), (1,), torch.bfloat16, "cpu")
        return tccl_amd.one_shot_all_reduce(t)          # 10 elements: not a multiple of the reference's 4

    with pytest.raises(AssertionError, match="128-bit aligned"):
        spmd.run(2, main)


def test_outside_run():
    with pytest.raises(RuntimeError, match="spmd.run"):
        spmd.empty_strided_p2p((8,), (1,), torch.bfloat16, "cpu")
    assert spmd.rendezvous_barrier() == 0
    with spmd.collective() as turn:
        assert turn.first
    with pytest.raises(ValueError, match="contiguous"):
        spmd.run(1, lambda r, w: spmd.empty_strided_p2p((4, 4), (1, 4), torch.float32, "cpu"))
