"""The reference's four ``__main__`` self-tests, rank program by rank program, run for W
virtual ranks on one GPU.  Where the reference compares with a bf16-stepwise CPU sum the
expected value here is the fp32-accumulate oracle (the arithmetic contract); the distance to
the reference's own expected value is checked to be what rounding differences allow."""
import pytest
import torch

import tccl_amd
from tccl_amd import spmd
from helpers import assert_bit_equal
from oracle import torch_ref

pytestmark = pytest.mark.gpu
WORLD = 8


def test_one_shot_all_reduce_main():
    """triton_one_shot_all_reduce_no_128.py:99-129."""
    def main(rank, world_size):
        device = torch.device("cuda:0")
        tensor = spmd.empty_strided_p2p(size=(8192,), stride=(1,), dtype=torch.bfloat16, device=device,
                                        group_name="world").fill_(rank)
        output = tccl_amd.one_shot_all_reduce(tensor)
        assert output.eq(world_size * (world_size - 1) // 2).all().item()
        return output.cpu()

    outs = spmd.run(WORLD, main)
    assert all(o.eq(28).all() for o in outs)


def _seeded_answers(size, world_size):
    """triton_reduce_scatter.py:197-200: the reference's expected value, a bf16 running sum."""
    answer = torch.zeros(size, dtype=torch.bfloat16)
    bufs = []
    for i in range(world_size):
        torch.manual_seed(i)
        bufs.append(torch.randn(size, dtype=torch.bfloat16))
        answer += bufs[-1]
    return bufs, answer


def test_reduce_scatter_main():
    """triton_reduce_scatter.py:175-211 at 1 Mi elements (the reference uses 256 Mi)."""
    size = 1 << 20

    def main(rank, world_size):
        device = torch.device("cuda:0")
        # the ranks are threads of one process here, so each takes its own generator where
        # the reference seeds the process-wide one (torch.manual_seed(rank), :185); the
        # numbers drawn are the same
        gen = torch.Generator().manual_seed(rank)
        tensor = spmd.empty_strided_p2p(size=(size,), stride=(1,), dtype=torch.bfloat16, device=device,
                                        group_name="world")
        tensor.copy_(torch.randn(size, dtype=torch.bfloat16, generator=gen))   # made on the CPU, as :189-195
        output = tccl_amd.one_shot_reduce_scatter(tensor)
        return output.cpu()

    outs = spmd.run(WORLD, main)
    bufs, stepwise = _seeded_answers(size, WORLD)
    contract = torch_ref.all_reduce(bufs)
    per = size // WORLD
    for rank, out in enumerate(outs):
        assert_bit_equal(out, contract[per * rank:per * (rank + 1)], f"rank {rank}")
        # the reference's own expected value re-rounds after every rank: same to within the
        # rounding of W bf16 additions
        ref = stepwise[per * rank:per * (rank + 1)].float()
        err = (out.float() - ref).abs()
        assert (err <= 2.0 ** -7 * WORLD * torch.maximum(ref.abs(), torch.tensor(8.0))).all()


def test_all_gather_main():
    """triton_all_gather.py:99-136 (the known-answer version kept in comments there)."""
    def main(rank, world_size):
        device = torch.device("cuda:0")
        tensor = spmd.empty_strided_p2p(size=(2048,), stride=(1,), dtype=torch.bfloat16, device=device,
                                        group_name="world").fill_(rank)
        output = tccl_amd.one_shot_all_gather(tensor, world_size)
        answer = torch.stack([torch.full((2048,), r, dtype=torch.bfloat16) for r in range(world_size)])
        assert torch.allclose(output.cpu(), answer)
        return output.cpu()

    outs = spmd.run(WORLD, main)
    for o in outs[1:]:
        assert_bit_equal(o, outs[0], "all ranks gather the same")


@pytest.mark.parametrize("fused", [False, True, "pipelined"])
def test_double_tree_all_reduce_main(fused):
    """triton_double_tree_allreduce.py:373-410: 8,192 seeded elements per rank.  The
    reference compares with the flat bf16 running sum (its kernel never produced the value);
    here the expected value is the tree-ordered oracle, and the flat sum is only close."""
    size = 8192

    def main(rank, world_size):
        device = torch.device("cuda:0")
        gen = torch.Generator().manual_seed(rank)
        tensor = spmd.empty_strided_p2p(size=(size,), stride=(1,), dtype=torch.bfloat16, device=device,
                                        group_name="world")
        tensor.copy_(torch.randn(size, dtype=torch.bfloat16, generator=gen))
        if fused == "pipelined":        # the reference kernel's own design: wait, reduce, send
            output = tccl_amd.double_tree_all_reduce(tensor, pipelined=True)
        else:
            output = tccl_amd.double_tree_all_reduce(tensor, fused=fused)
        return output.cpu(), tensor.cpu()

    results = spmd.run(WORLD, main)
    bufs, stepwise = _seeded_answers(size, WORLD)
    want = torch_ref.double_tree_all_reduce(bufs)[0]
    for rank, (out, buf) in enumerate(results):
        assert_bit_equal(out, want, f"output of rank {rank}")
        assert_bit_equal(buf, want, f"buffer of rank {rank} after the collective")
    assert torch.allclose(want.float(), stepwise.float(), rtol=0.05, atol=0.25)


def test_two_collectives_back_to_back_do_not_race():
    """A rank refills its buffer right after a collective returns: the trailing rendezvous
    keeps that write behind every peer's read."""
    def main(rank, world_size):
        tensor = spmd.empty_strided_p2p((1 << 16,), (1,), torch.bfloat16, "cuda:0").fill_(rank)
        first = tccl_amd.one_shot_all_reduce(tensor)
        tensor.fill_(1)
        second = tccl_amd.one_shot_all_reduce(tensor)
        third = tccl_amd.two_shot_all_reduce(tensor)
        return first.cpu(), second.cpu(), third.cpu()

    for first, second, third in spmd.run(WORLD, main):
        assert first.eq(28).all() and second.eq(WORLD).all() and third.eq(WORLD).all()
