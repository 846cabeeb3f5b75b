"""Seeded random cases on the GPU: every entry point with random worlds, sizes, dtypes and
launch overrides against the C oracle, bit for bit.  The case list is fixed by the seed, so
a failure names a reproducible case."""
import ctypes

import numpy as np
import pytest
import torch

import tccl_amd
from tccl_amd import _lib
from helpers import assert_bit_equal, from_np_bits, np_bits
from oracle import torch_ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        world = int(rng.integers(1, 9))
        dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float32
        per_vec = 16 // (2 if dtype == torch.bfloat16 else 4)
        scale = int(rng.choice([1, 1, 1, 40, 40, 700, 9000]))
        nvec = int(rng.integers(0, 1 + 97 * scale))
        ragged = int(rng.integers(0, per_vec)) if rng.random() < 0.4 else 0
        flags = int(rng.choice([0, 0, 1, 2, 3, 4, 16, 16 | 3, 32, 32, 32]))
        cfg = dict(block=int(rng.choice([0, 64, 128, 256, 512])), unroll=int(rng.choice([0, 1, 2, 4, 8])),
                   grid=int(rng.choice([0, 0, 1, 3, 8, 64, 1000])), tile_iters=int(rng.choice([0, 0, 1, 2, 5, 16, 32])),
                   flags=flags)
        out.append((i, world, dtype, nvec * per_vec + ragged, cfg))
    return out


def _inputs(world, numel, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    n = max(numel, 1)
    if dtype == torch.bfloat16:
        return [torch.randn(n, generator=g).to(torch.bfloat16) for _ in range(world)]
    return [torch.rand(n, generator=g) * 2 - 1 for _ in range(world)]


def _oracle(c_oracle, bufs):
    if bufs[0].dtype == torch.bfloat16:
        return from_np_bits(c_oracle.all_reduce_bf16([np_bits(b) for b in bufs]))
    return torch.from_numpy(c_oracle.all_reduce_f32([b.numpy() for b in bufs]))


def _default_plan_cases(n, seed):
    """Sizes across every launch plan the library chooses by itself (no launch overrides): the
    grid-stride kernel, the plan for small inputs, partial and full tiles, unequal interleaved
    tiles, several launches per call, the single-launch rule for few sources."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        world = int(rng.integers(1, 9))
        dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float32
        esize = 2 if dtype == torch.bfloat16 else 4
        mib = float(rng.choice([1.7, 2.0, 2.3, 3.1, 4.0, 4.6, 6.5, 8.0, 8.1, 13.0, 24.0, 31.9, 32.0, 47.0, 63.9, 64.0, 65.0, 100.0]))
        numel = int(mib * (1 << 20)) // esize + int(rng.integers(-40, 41))
        out.append((i, world, dtype, numel))
    return out


@pytest.mark.parametrize("case", _default_plan_cases(36, 77), ids=lambda c: f"plan{c[0]}")
def test_random_sizes_default_plans(case, c_oracle):
    i, world, dtype, numel = case
    lib = tccl_amd.load_library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator().manual_seed(5000 + i)
    first = torch.randn(numel, generator=g).to(dtype) if dtype == torch.bfloat16 else torch.rand(numel, generator=g) * 2 - 1
    bufs = [first.roll(r * 7919) for r in range(world)]
    dev = [b.to(DEV) for b in bufs]
    ptrs = _lib.ptr_array([d.data_ptr() for d in dev])
    dt = _lib.TCCL_BF16 if dtype == torch.bfloat16 else _lib.TCCL_F32
    out = torch.full((numel + 32,), 3.0, dtype=dtype, device=DEV)
    print(f"plan case {i}: world={world} dtype={dtype} numel={numel}", flush=True)
    assert lib.tccl_all_reduce_sum(ptrs, world, out.data_ptr(), numel, dt, stream) == 0
    assert_bit_equal(out[:numel], _oracle(c_oracle, bufs), "all-reduce")
    assert out[numel:].eq(3.0).all().item(), "wrote past the end"


@pytest.mark.parametrize("case", _cases(80, 20240607), ids=lambda c: f"case{c[0]}")
def test_random_all_reduce_and_reduce_scatter(case, c_oracle):
    i, world, dtype, numel, cfgd = case
    lib = tccl_amd.load_library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    bufs = _inputs(world, numel, dtype, 1000 + i)
    dev = [b.to(DEV) for b in bufs]
    ptrs = _lib.ptr_array([d.data_ptr() for d in dev])
    dt = _lib.TCCL_BF16 if dtype == torch.bfloat16 else _lib.TCCL_F32
    cfg = tccl_amd.LaunchCfg(**cfgd)
    out = torch.full((numel + 32,), 3.0, dtype=dtype, device=DEV)
    print(f"case {i}: world={world} dtype={dtype} numel={numel} cfg={cfgd}", flush=True)
    assert lib.tccl_all_reduce_sum_ex(ptrs, world, out.data_ptr(), numel, dt, stream, ctypes.byref(cfg)) == 0
    want = _oracle(c_oracle, [b[:numel].contiguous() for b in bufs]) if numel else bufs[0][:0]
    assert_bit_equal(out[:numel], want, "all-reduce")
    assert out[numel:].eq(3.0).all().item(), "wrote past the end"
    # reduce-scatter of the same buffers for a random rank, when the share is vector-aligned
    per_vec = 16 // bufs[0].element_size()
    total = (numel // (per_vec * world)) * per_vec * world
    if total:
        rank = i % world
        per = total // world
        share = torch.full((per + 32,), 3.0, dtype=dtype, device=DEV)
        assert lib.tccl_reduce_scatter_sum_ex(ptrs, world, rank, share.data_ptr(), total, dt, stream,
                                              ctypes.byref(cfg)) == 0
        w = _oracle(c_oracle, [b[rank * per:(rank + 1) * per].contiguous() for b in bufs])
        assert_bit_equal(share[:per], w, "reduce-scatter")
        assert share[per:].eq(3.0).all().item()


@pytest.mark.parametrize("case", _cases(40, 77), ids=lambda c: f"case{c[0]}")
def test_random_all_gather_and_tree_steps(case, c_oracle):
    i, world, dtype, numel, cfgd = case
    lib = tccl_amd.load_library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    per_vec = 16 // (2 if dtype == torch.bfloat16 else 4)
    numel = numel // per_vec * per_vec                       # copies take whole vectors only
    bufs = _inputs(world, numel, dtype, 5000 + i)
    dev = [b[:numel].contiguous().to(DEV) for b in bufs]
    print(f"case {i}: world={world} dtype={dtype} numel={numel} cfg={cfgd}", flush=True)
    if numel:
        ptrs = _lib.ptr_array([d.data_ptr() for d in dev])
        cfgd = dict(cfgd, unroll=cfgd["unroll"] if cfgd["unroll"] != 8 else 4, flags=cfgd["flags"] & 15)
        cfg = tccl_amd.LaunchCfg(**cfgd)
        out = torch.zeros((world, numel), dtype=dtype, device=DEV)
        nbytes = numel * bufs[0].element_size()
        assert lib.tccl_all_gather_ex(ptrs, world, out.data_ptr(), nbytes, stream, ctypes.byref(cfg)) == 0
        assert_bit_equal(out, torch.stack([b[:numel] for b in bufs]), "all-gather")
    if not numel:
        return
    # one tree reduce step with the children this case's world allows, in place
    dt = _lib.TCCL_BF16 if dtype == torch.bfloat16 else _lib.TCCL_F32
    own = bufs[0][:numel].contiguous()
    c0 = bufs[1][:numel].contiguous() if world >= 2 and i % 2 == 0 else None
    c1 = bufs[2][:numel].contiguous() if world >= 3 and i % 3 != 0 else None
    d_own = own.to(DEV)
    d0 = c0.to(DEV) if c0 is not None else None
    d1 = c1.to(DEV) if c1 is not None else None
    rc = lib.tccl_tree_reduce_step(d_own.data_ptr(), d0.data_ptr() if d0 is not None else None,
                                   d1.data_ptr() if d1 is not None else None, d_own.data_ptr(), numel, dt, stream)
    assert rc == 0
    assert_bit_equal(d_own, torch_ref.tree_reduce_step(own, c0, c1), "tree reduce step in place")
    # and the copy step into two destinations
    a = torch.zeros_like(d_own)
    b = torch.zeros_like(d_own)
    assert lib.tccl_tree_copy_step(d_own.data_ptr(), a.data_ptr(), b.data_ptr(), numel * own.element_size(),
                                   stream) == 0
    assert_bit_equal(a, d_own, "copy dst0")
    assert_bit_equal(b, d_own, "copy dst1")


def _signalling_cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float32
        per_vec = 16 // (2 if dtype == torch.bfloat16 else 4)
        scale = int(rng.choice([1, 1, 40, 700, 9000, 60000]))
        nvec = int(rng.integers(1, 2 + 97 * scale))
        chunk_vecs = int(rng.choice([0, 0, 0, 1, 3, 64, 1000, 2048, 8192, 20000]))
        pcfg = dict(workgroups=int(rng.choice([0, 0, 0, 8, 24, 100, 333, 1000, 5000])), lag=int(rng.choice([0, 1, 2, 4])),
                    tile_kib=int(rng.choice([0, 32, 128])))
        out.append((i, int(rng.choice([2, 4, 8])), int(rng.integers(1, 9)), dtype, nvec * per_vec, chunk_vecs * per_vec,
                    pcfg))
    return out


@pytest.mark.parametrize("case", _signalling_cases(40, 20240611), ids=lambda c: f"case{c[0]}")
def test_random_signalling_kernels(case, c_oracle):
    """The pipelined double tree (random power-of-two world, chunk size, grid, lag, tile) and
    the one-launch two-shot (random world 1..8, grid) against the oracles, with no expired
    wait and clean pads afterwards."""
    i, tree_world, flat_world, dtype, numel, chunk_elems, pcfgd = case
    print(f"signalling case {i}: {case[1:]}", flush=True)
    pcfg = _lib.PipelineCfg(spin_limit=1 << 18, **pcfgd)
    pcfg.flags = _lib.PIPE_DRAW_PLACES if i % 2 else 0          # both ways of binding places to workgroups
    # pipelined double tree
    bufs = _inputs(tree_world, numel, dtype, 3000 + i)
    want = torch_ref.double_tree_all_reduce(bufs)[0]
    g = tccl_amd.empty_world(tree_world, numel, dtype, DEV)
    try:
        for r, b in enumerate(bufs):
            g.tensor(r).copy_(b)
        outs = tccl_amd.double_tree_all_reduce_world(g, pipelined=True, chunk_elems=chunk_elems, pipeline_cfg=pcfg)
        assert tccl_amd.signal_pad_timeouts(g) == 0
        for r in range(tree_world):
            assert_bit_equal(outs[r], want, f"case {i}: tree output {r}")
            assert_bit_equal(g.tensor(r), want, f"case {i}: tree buffer {r}")
        assert all(int(p.count_nonzero().item()) == 0 for p in g._signal_pads)   # noqa: SLF001
    finally:
        tccl_amd.unregister(g)
    # one-launch two-shot: every share whole vectors
    per_vec = 16 // bufs[0].element_size()
    numel2 = max(numel // (per_vec * flat_world), 1) * per_vec * flat_world
    bufs = _inputs(flat_world, numel2, dtype, 4000 + i)
    want = _oracle(c_oracle, bufs)
    g = tccl_amd.empty_world(flat_world, numel2, dtype, DEV)
    try:
        for r, b in enumerate(bufs):
            g.tensor(r).copy_(b)
        outs = tccl_amd.two_shot_all_reduce_world(g, with_outputs=(i % 2 == 0), pipeline_cfg=pcfg)
        assert tccl_amd.signal_pad_timeouts(g) == 0
        for r in range(flat_world):
            if outs is not None:
                assert_bit_equal(outs[r], want, f"case {i}: two-shot output {r}")
            assert_bit_equal(g.tensor(r), want, f"case {i}: two-shot buffer {r}")
        assert all(int(p.count_nonzero().item()) == 0 for p in g._signal_pads)   # noqa: SLF001
    finally:
        tccl_amd.unregister(g)
