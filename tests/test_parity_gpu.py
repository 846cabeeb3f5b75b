"""GPU parity: every HIP kernel, called through the C ABI (directly or via the host
wrappers, which only add allocation and argument checks), against the CPU oracle on the
same seeded inputs.  Bit-exact unless stated."""
import ctypes
import gc

import numpy as np
import pytest
import torch

import tccl_amd
from tccl_amd import _lib
from helpers import (assert_bit_equal, assert_bit_equal_nan_aware, from_np_bits, np_bits, seeded_int8,
                     seeded_randn, seeded_uniform)
from oracle import torch_ref

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _gpu_hygiene():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    tccl_amd.load_library()
    groups = []
    yield groups
    torch.cuda.synchronize()
    for g in groups:
        tccl_amd.unregister(g)
    groups.clear()
    gc.collect()
    torch.cuda.empty_cache()


def upload(groups, bufs):
    """One separate device allocation per virtual rank, filled from the CPU tensors."""
    g = tccl_amd.empty_world(len(bufs), bufs[0].shape, bufs[0].dtype, DEV)
    for r, b in enumerate(bufs):
        g.tensor(r).copy_(b)
    groups.append(g)
    return g


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def oracle_sum(c_oracle, bufs):
    if bufs[0].dtype == torch.bfloat16:
        return from_np_bits(c_oracle.all_reduce_bf16([np_bits(b) for b in bufs]))
    return torch.from_numpy(c_oracle.all_reduce_f32([b.numpy() for b in bufs]))


# ------------------------------------------------------------------ one-shot all-reduce

@pytest.mark.parametrize("world", [2, 4, 8])
def test_all_reduce_fill_rank(world, _gpu_hygiene):
    """The reference's own test, triton_one_shot_all_reduce_no_128.py:116-127."""
    g = upload(_gpu_hygiene, [torch.full((8192,), float(r), dtype=torch.bfloat16) for r in range(world)])
    for r in range(world):
        out = tccl_amd.one_shot_all_reduce(g.tensor(r))
        assert out.eq(world * (world - 1) // 2).all().item()
        assert out.dtype == torch.bfloat16 and out.shape == (8192,)


@pytest.mark.parametrize("world", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform], ids=["bf16", "f32"])
def test_all_reduce_matches_oracle(world, maker, _gpu_hygiene, c_oracle):
    numel = 8 * 40_003                       # many tiles plus a partial one
    bufs = maker(world, numel)
    g = upload(_gpu_hygiene, bufs)
    want = oracle_sum(c_oracle, bufs)
    assert_bit_equal(tccl_amd.one_shot_all_reduce(g.tensor(0)), want, f"W={world}")


@pytest.mark.parametrize("numel", [0, 1, 7, 8, 9, 515, 2048 * 8 + 5, 1_000_003])
@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform], ids=["bf16", "f32"])
def test_all_reduce_ragged_sizes_through_c_abi(numel, maker, _gpu_hygiene, c_oracle):
    """Sizes that are not whole 16-byte vectors: the wrappers refuse them as the reference
    does, the C entry point sums the tail one element at a time."""
    world = 4
    bufs = maker(world, max(numel, 8))
    g = upload(_gpu_hygiene, bufs)
    out = torch.full((max(numel, 8) + 8,), 77.0, dtype=bufs[0].dtype, device=DEV)
    dt = _lib.TCCL_BF16 if bufs[0].dtype == torch.bfloat16 else _lib.TCCL_F32
    rc = tccl_amd.load_library().tccl_all_reduce_sum(g.ptr_array, world, out.data_ptr(), numel, dt, stream())
    assert rc == 0
    want = oracle_sum(c_oracle, [b[:numel].contiguous() for b in bufs]) if numel else bufs[0][:0]
    assert_bit_equal(out[:numel], want, f"numel={numel}")
    assert out[numel:].eq(77.0).all().item(), "wrote past the end"


@pytest.mark.parametrize("block", [64, 128, 256, 512])
@pytest.mark.parametrize("unroll", [1, 2, 4])
@pytest.mark.parametrize("flags", [0, 1, 2, 3, 4, 7])
def test_all_reduce_every_launch_shape(block, unroll, flags, _gpu_hygiene, c_oracle):
    """Every kernel instantiation and tiling mode gives the same bits."""
    bufs = seeded_randn(8, 8 * 30_011)
    g = upload(_gpu_hygiene, bufs)
    want = oracle_sum(c_oracle, bufs)
    for tile_iters, grid in ((0, 0), (4, 0), (1, 24), (3, 40), (16, 8)):
        cfg = tccl_amd.LaunchCfg(block=block, unroll=unroll, grid=grid, tile_iters=tile_iters, flags=flags)
        got = tccl_amd.one_shot_all_reduce(g.tensor(0), cfg=cfg)
        assert_bit_equal(got, want, f"block={block} unroll={unroll} flags={flags} tile={tile_iters} grid={grid}")
    small = seeded_randn(3, 8 * 1001)
    g3 = upload(_gpu_hygiene, small)
    cfg = tccl_amd.LaunchCfg(block=block, unroll=unroll, flags=flags)
    assert_bit_equal(tccl_amd.one_shot_all_reduce(g3.tensor(0), cfg=cfg), oracle_sum(c_oracle, small), "W=3")


@pytest.mark.parametrize("world", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform], ids=["bf16", "f32"])
def test_all_reduce_phased_kernel_forced(world, maker, _gpu_hygiene, c_oracle):
    """The read-then-write kernel that large inputs take, forced onto small inputs so that
    partial tiles, several launches per call, every tile length and ragged tails are all
    exercised against the oracle."""
    per_vec = 8 if maker is seeded_randn else 4
    numel = per_vec * 100_003 + 3                      # not a whole number of vectors
    bufs = maker(world, numel + per_vec)
    g = upload(_gpu_hygiene, bufs)
    want = oracle_sum(c_oracle, [b[:numel].contiguous() for b in bufs])
    dt = _lib.TCCL_BF16 if bufs[0].dtype == torch.bfloat16 else _lib.TCCL_F32
    lib = tccl_amd.load_library()
    for tile_iters, grid in ((0, 0), (1, 0), (1, 7), (2, 3), (3, 16), (4, 512), (5, 1), (8, 2), (16, 4), (16, 1)):
        cfg = tccl_amd.LaunchCfg(grid=grid, tile_iters=tile_iters, flags=_lib.CFG_PHASED)
        out = torch.full((numel + 16,), 55.0, dtype=bufs[0].dtype, device=DEV)
        rc = lib.tccl_all_reduce_sum_ex(g.ptr_array, world, out.data_ptr(), numel, dt, stream(), ctypes.byref(cfg))
        assert rc == 0
        assert_bit_equal(out[:numel], want, f"W={world} K={tile_iters} grid={grid}")
        assert out[numel:].eq(55.0).all().item(), "wrote past the end"
    # sizes below one vector and exactly one tile
    for n in (0, 1, per_vec - 1, per_vec, 256 * per_vec * 2, 256 * per_vec * 2 * 16 + 1):
        cfg = tccl_amd.LaunchCfg(flags=_lib.CFG_PHASED)
        out = torch.full((n + 16,), 55.0, dtype=bufs[0].dtype, device=DEV)
        assert lib.tccl_all_reduce_sum_ex(g.ptr_array, world, out.data_ptr(), n, dt, stream(), ctypes.byref(cfg)) == 0
        w = oracle_sum(c_oracle, [b[:n].contiguous() for b in bufs]) if n else bufs[0][:0]
        assert_bit_equal(out[:n], w, f"W={world} n={n}")
        assert out[n:].eq(55.0).all().item()


def test_phased_and_streaming_kernels_agree_at_headline_size(_gpu_hygiene, c_oracle):
    """W=8 x 64 MiB bf16: default dispatch (phased), forced streaming, and the oracle."""
    n = (64 << 20) // 2
    bufs = seeded_randn(8, n)
    g = upload(_gpu_hygiene, bufs)
    want = oracle_sum(c_oracle, bufs)
    assert_bit_equal(tccl_amd.one_shot_all_reduce(g.tensor(0)), want, "default")
    for flags in (_lib.CFG_STREAMING | 3, _lib.CFG_PHASED):
        cfg = tccl_amd.LaunchCfg(flags=flags)
        assert_bit_equal(tccl_amd.one_shot_all_reduce(g.tensor(0), cfg=cfg), want, f"flags={flags}")


@pytest.mark.parametrize("world,mib", [(8, 2), (3, 2), (8, 4), (4, 4), (8, 8), (4, 8), (2, 8), (8, 32), (4, 32), (3, 32), (8, 64),
                                       (5, 64), (4, 64), (3, 64), (3, 96), (2, 48), (1, 48), (1, 4)])
def test_all_reduce_around_dispatch_thresholds(world, mib, _gpu_hygiene, c_oracle):
    """Sizes one vector below, at, one vector above and raggedly above every size at which
    the library changes kernel or launch plan (grid-stride -> phased at 2 or 4 MiB of output, the
    plan for small inputs up to 8 MiB and its switch to more vectors per iteration, full tiles
    -- and with them unequal, interleaved tiles -- for one workgroup per compute unit at 32 MiB
    and for two at 64 MiB, the single-launch rule for few sources at 48/96 MiB)."""
    base = (mib << 20) // 2
    top = base + 8 * 1025 + 3
    torch.manual_seed(world * 1000 + mib)
    first = torch.randn(top, dtype=torch.bfloat16)
    bufs = [first.roll(r * 104_729) for r in range(world)]
    g = upload(_gpu_hygiene, bufs)
    lib = tccl_amd.load_library()
    out = torch.empty(top + 64, dtype=torch.bfloat16, device=DEV)
    for numel in (base - 8, base, base + 8, base + 8 * 1025 + 3):
        out.fill_(9.0)
        assert lib.tccl_all_reduce_sum(g.ptr_array, world, out.data_ptr(), numel, _lib.TCCL_BF16, stream()) == 0
        want = oracle_sum(c_oracle, [b[:numel].contiguous() for b in bufs])
        assert_bit_equal(out[:numel], want, f"W={world} numel={numel}")
        assert out[numel:numel + 64].eq(9.0).all().item(), "wrote past the end"


def test_all_reduce_wrapper_takes_multiples_of_four_elements(_gpu_hygiene, c_oracle):
    """The reference's wrapper accepts any multiple of 4 bf16 elements
    (triton_one_shot_all_reduce_no_128.py:70-76), not only whole 16-byte vectors."""
    bufs = seeded_randn(8, 8 * 1000 + 4)
    g = upload(_gpu_hygiene, bufs)
    for numel in (4, 12, 8 * 1000 + 4):
        got = tccl_amd.one_shot_all_reduce(g.tensor(0)[:numel])
        assert_bit_equal(got, oracle_sum(c_oracle, [b[:numel].contiguous() for b in bufs]), f"numel={numel}")


@pytest.mark.parametrize("world", [3, 4, 8])
def test_all_reduce_f32_full_tiles(world, _gpu_hygiene, c_oracle):
    """fp32 where the input is cut into full tiles (unequal, interleaved tiles for three sources
    or more): exactly one wave of tiles, one element less, and a ragged size above it."""
    base = (64 << 20) // 4
    top = base + 4 * 1025 + 3
    bufs = seeded_uniform(world, top, seed_base=40 + world)
    g = upload(_gpu_hygiene, bufs)
    lib = tccl_amd.load_library()
    out = torch.empty(top + 64, dtype=torch.float32, device=DEV)
    for numel in (base - 1, base, top):
        out.fill_(9.0)
        assert lib.tccl_all_reduce_sum(g.ptr_array, world, out.data_ptr(), numel, _lib.TCCL_F32, stream()) == 0
        want = oracle_sum(c_oracle, [b[:numel].contiguous() for b in bufs])
        assert_bit_equal(out[:numel], want, f"W={world} numel={numel}")
        assert out[numel:numel + 64].eq(9.0).all().item(), "wrote past the end"


def test_all_reduce_order_and_single_rounding(_gpu_hygiene):
    """fp32 accumulation in rank order: [2^24, 1 x6, -2^24] -> 0; ones first -> 6;
    1 + 2^-8 + 2^-8 -> 1 + 2^-7 (a bf16-stepwise sum would give 1)."""
    vals = [2.0 ** 24, 1, 1, 1, 1, 1, 1, -(2.0 ** 24)]
    for dtype in (torch.bfloat16, torch.float32):
        g = upload(_gpu_hygiene, [torch.full((4096,), v, dtype=dtype) for v in vals])
        assert tccl_amd.one_shot_all_reduce(g.tensor(0)).eq(0).all().item()
        rot = upload(_gpu_hygiene, [torch.full((4096,), vals[i], dtype=dtype) for i in (1, 2, 3, 4, 5, 6, 0, 7)])
        assert tccl_amd.one_shot_all_reduce(rot.tensor(0)).eq(6).all().item()
    g = upload(_gpu_hygiene, [torch.full((4096,), v, dtype=torch.bfloat16) for v in (1.0, 2.0 ** -8, 2.0 ** -8)])
    assert tccl_amd.one_shot_all_reduce(g.tensor(0)).float().eq(1.0 + 2.0 ** -7).all().item()


def test_all_reduce_directed_bit_patterns(_gpu_hygiene, c_oracle):
    """Subnormals (kept, not flushed), signed zeros (+0 start), infinities, overflow to
    infinity, round-to-nearest-even ties, NaN (any NaN encoding accepted)."""
    pats = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x7F7F, 0xFF7F, 0x7F80, 0xFF80, 0x3F80,
                     0xBF80, 0x3F81, 0x4B80, 0xCB80, 0x3380, 0x0100, 0x8100, 0x7FC0, 0xFFC1], dtype=np.uint16)
    rng = np.random.default_rng(5)
    for world in (2, 3, 8):
        bufs = [from_np_bits(pats[rng.integers(0, len(pats), size=8 * 4096)]) for _ in range(world)]
        g = upload(_gpu_hygiene, bufs)
        want = oracle_sum(c_oracle, bufs)
        assert_bit_equal_nan_aware(tccl_amd.one_shot_all_reduce(g.tensor(0)), want, f"W={world}")
    # ties: 1 + 2^-8 is halfway between bf16 1.0 and 1+2^-7 -> even (1.0); 1+2^-7 + 2^-8 -> 1+2^-6
    for base, want in ((1.0, 1.0), (1.0 + 2.0 ** -7, 1.0 + 2.0 ** -6)):
        g = upload(_gpu_hygiene, [torch.full((64,), base, dtype=torch.bfloat16),
                                  torch.full((64,), 2.0 ** -8, dtype=torch.bfloat16)])
        assert tccl_amd.one_shot_all_reduce(g.tensor(0)).float().eq(want).all().item()
    # -0 + -0 -> +0 because the accumulator starts at +0
    g = upload(_gpu_hygiene, [torch.full((64,), -0.0, dtype=torch.bfloat16) for _ in range(2)])
    assert np.array_equal(np_bits(tccl_amd.one_shot_all_reduce(g.tensor(0))), np.zeros(64, np.uint16))
    # fp32 subnormals survive
    tiny = torch.full((64,), 1e-45, dtype=torch.float32)
    g = upload(_gpu_hygiene, [tiny.clone(), tiny.clone()])
    assert_bit_equal(tccl_amd.one_shot_all_reduce(g.tensor(0)), tiny + tiny, "fp32 subnormal")


def test_all_reduce_config1_vs_torch_cpu_reference(_gpu_hygiene, c_oracle):
    """Benchmark shape 1: W=8 x 4,194,304 bf16 ~N(0,1), seed = rank, against the torch CPU
    reference (and the C oracle)."""
    bufs = seeded_randn(8, 4_194_304)
    g = upload(_gpu_hygiene, bufs)
    want = torch_ref.all_reduce(bufs)
    for r in (0, 5):
        assert_bit_equal(tccl_amd.one_shot_all_reduce(g.tensor(r)), want, f"rank {r}")
    assert_bit_equal(oracle_sum(c_oracle, bufs), want, "oracles")


@pytest.mark.parametrize("world", [2, 4, 8])
def test_all_reduce_sweep_sizes(world, _gpu_hygiene, c_oracle):
    """Benchmark sweep (shape 2): 16 KiB .. 64 MiB per buffer in powers of 4, using prefix
    views of one allocation (as the reference's benchmarks slice tensor[:size])."""
    top = (64 << 20) // 2
    bufs = seeded_randn(world, top)
    g = upload(_gpu_hygiene, bufs)
    nbytes = 16 << 10
    while nbytes <= (64 << 20):
        n = nbytes // 2
        want = oracle_sum(c_oracle, [b[:n] for b in bufs])
        assert_bit_equal(tccl_amd.one_shot_all_reduce(g.tensor(1)[:n]), want, f"W={world} {nbytes} B")
        nbytes *= 4


@pytest.mark.parametrize("world", [2, 4, 8])
def test_all_reduce_256mib_per_buffer(world, _gpu_hygiene, c_oracle):
    """Largest sweep point for every world of the sweep: W x 256 MiB against the oracle (offsets
    beyond 2^31 bytes in total at W=8; at W=2 the launch plan is the one for few sources: a single
    launch over 16 KiB tiles; at W=4 and 8, four and four slices of full-size tiles)."""
    n = (256 << 20) // 2
    torch.manual_seed(0)
    base = torch.randn(n, dtype=torch.bfloat16)
    bufs = [base.roll(r * 1_000_003) for r in range(world)]
    g = upload(_gpu_hygiene, bufs)
    out = tccl_amd.one_shot_all_reduce(g.tensor(world - 1))
    want = oracle_sum(c_oracle, bufs)
    assert_bit_equal(out, want, f"W={world} x 256 MiB")


def test_launches_follow_the_current_stream(_gpu_hygiene, c_oracle):
    """Kernels go to torch's current stream: producer work queued on a side stream is seen
    by the collective launched after it on that stream, with no device synchronisation in
    between, and the default stream learns of the result through an event."""
    world, numel = 8, 8 * 8 * 37_501
    bufs = seeded_randn(world, numel, seed_base=77)
    want = oracle_sum(c_oracle, bufs)
    g = tccl_amd.empty_world(world, numel, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    staged = [b.to(DEV) for b in bufs]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for r in range(world):
            g.tensor(r).zero_()
            g.tensor(r).copy_(staged[r], non_blocking=True)     # producer, on the side stream
        out = tccl_amd.one_shot_all_reduce(g.tensor(0))          # consumer, same stream
        share = tccl_amd.reduce_scatter(g.tensor(1))
        done = torch.cuda.Event()
        done.record(side)
    torch.cuda.current_stream().wait_event(done)
    doubled = out.float() * 2                                    # default-stream consumer
    torch.cuda.synchronize()
    assert_bit_equal(out, want, "side stream")
    per = numel // world
    assert_bit_equal(share, want[per:2 * per], "side stream reduce-scatter")
    assert torch.equal(doubled.cpu(), want.float() * 2)


def test_caller_provided_outputs(_gpu_hygiene, c_oracle):
    world, numel = 4, 8 * 4 * 5_003
    bufs = seeded_randn(world, numel, seed_base=61)
    g = upload(_gpu_hygiene, bufs)
    want = oracle_sum(c_oracle, bufs)
    per = numel // world
    out = torch.empty(numel, dtype=torch.bfloat16, device=DEV)
    share = torch.empty(per, dtype=torch.bfloat16, device=DEV)
    rows = torch.empty((world, numel), dtype=torch.bfloat16, device=DEV)
    assert tccl_amd.one_shot_all_reduce(g.tensor(0), out=out) is out
    assert tccl_amd.reduce_scatter(g.tensor(2), out=share) is share
    assert tccl_amd.all_gather(g.tensor(0), world, out=rows) is rows
    assert_bit_equal(out, want, "all-reduce into out")
    assert_bit_equal(share, want[2 * per:3 * per], "reduce-scatter into out")
    assert_bit_equal(rows, torch.stack(bufs), "all-gather into out")
    for bad in (torch.empty(numel + 8, dtype=torch.bfloat16, device=DEV), torch.empty(numel, dtype=torch.float32, device=DEV),
                torch.empty(2 * numel, dtype=torch.bfloat16, device=DEV)[::2]):
        with pytest.raises(ValueError, match="out must be"):
            tccl_amd.one_shot_all_reduce(g.tensor(0), out=bad)


def test_concurrent_callers_on_their_own_streams(_gpu_hygiene, c_oracle):
    """The library keeps no state between calls: four host threads, each with its own group
    and its own stream, call every operation at the same time."""
    import threading
    world, numel, threads = 4, 8 * 4 * 30_011, 4
    inputs = [seeded_randn(world, numel, seed_base=900 + 10 * t) for t in range(threads)]
    groups = [upload(_gpu_hygiene, inputs[t]) for t in range(threads)]
    torch.cuda.synchronize()
    results, errors = [None] * threads, []

    def work(t):
        try:
            torch.cuda.set_device(0)
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                acc = []
                for _ in range(20):
                    ar = tccl_amd.one_shot_all_reduce(groups[t].tensor(0))
                    rs = tccl_amd.reduce_scatter(groups[t].tensor(t % world))
                    ag = tccl_amd.all_gather(groups[t].tensor(0), world)
                    ts = tccl_amd.two_shot_all_reduce(groups[t].tensor(1))
                    acc.append((ar, rs, ag, ts))
                s.synchronize()
            results[t] = acc
        except BaseException as e:       # noqa: BLE001 -- reported below
            errors.append(e)

    pool = [threading.Thread(target=work, args=(t,)) for t in range(threads)]
    for p in pool:
        p.start()
    for p in pool:
        p.join()
    assert not errors, errors
    per = numel // world
    for t in range(threads):
        want = oracle_sum(c_oracle, inputs[t])
        for ar, rs, ag, ts in results[t][::7]:
            assert_bit_equal(ar, want, f"thread {t} all-reduce")
            assert_bit_equal(rs, want[(t % world) * per:(t % world + 1) * per], f"thread {t} reduce-scatter")
            assert_bit_equal(ag, torch.stack(inputs[t]), f"thread {t} all-gather")
            assert_bit_equal(ts, want, f"thread {t} two-shot")


def test_entry_points_can_be_captured_in_a_graph(_gpu_hygiene, c_oracle):
    """The entry points neither allocate nor synchronise, so a caller can record them into a
    HIP graph of its own (here through torch.cuda.graph) and replay it.  Replayed several
    times with new inputs and eager work in between; every replay is checked."""
    world, numel = 8, 8 * 8 * 20_001
    g = tccl_amd.empty_world(world, numel, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    lib = tccl_amd.load_library()
    out = torch.empty(numel, dtype=torch.bfloat16, device=DEV)
    share = torch.empty(numel // world, dtype=torch.bfloat16, device=DEV)
    gathered = torch.empty((world, numel), dtype=torch.bfloat16, device=DEV)

    def enqueue():
        s = stream()
        assert lib.tccl_all_reduce_sum(g.ptr_array, world, out.data_ptr(), numel, _lib.TCCL_BF16, s) == 0
        assert lib.tccl_reduce_scatter_sum(g.ptr_array, world, 5, share.data_ptr(), numel, _lib.TCCL_BF16, s) == 0
        assert lib.tccl_all_gather(g.ptr_array, world, gathered.data_ptr(), numel * 2, s) == 0

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue()                                  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    per = numel // world
    for rep in range(4):
        bufs = seeded_randn(world, numel, seed_base=500 + 10 * rep)
        for r in range(world):
            g.tensor(r).copy_(bufs[r])
        out.zero_(), share.zero_(), gathered.zero_()
        graph.replay()
        torch.cuda.synchronize()
        want = oracle_sum(c_oracle, bufs)
        assert_bit_equal(out, want, f"replay {rep} all-reduce")
        assert_bit_equal(share, want[5 * per:6 * per], f"replay {rep} reduce-scatter")
        assert_bit_equal(gathered, torch.stack(bufs), f"replay {rep} all-gather")
        assert_bit_equal(tccl_amd.one_shot_all_reduce(g.tensor(0)), want, f"eager after replay {rep}")


def test_buffers_larger_than_4_gib(_gpu_hygiene, c_oracle):
    """Offsets beyond 2^32 bytes inside ONE buffer: W=2 all-reduce over 2^31 + 98,760 bf16
    elements (4 GiB + 193 KiB per buffer), all-gather of the same rows, and a two-destination
    copy step.  Checked on the GPU in slices (with two sources the contract is exactly
    round(a + b)), and against the C oracle on windows around the 4 GiB mark and the end."""
    numel = (1 << 31) + 8 * 12_345
    g = tccl_amd.empty_world(2, numel, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    step = 1 << 28
    for r in range(2):
        gen = torch.Generator(device=DEV).manual_seed(40 + r)
        for lo in range(0, numel, step):
            n = min(step, numel - lo)
            g.tensor(r)[lo:lo + n].copy_(torch.randn(n, dtype=torch.float32, device=DEV, generator=gen))
    a, b = g.tensor(0), g.tensor(1)
    out = tccl_amd.one_shot_all_reduce(a)
    for lo in range(0, numel, step):
        n = min(step, numel - lo)
        want = (a[lo:lo + n].float() + b[lo:lo + n].float()).to(torch.bfloat16)
        assert torch.equal(out[lo:lo + n].view(torch.int16), want.view(torch.int16)), f"slice at {lo}"
    for lo, n in (((1 << 31) - 4096, 8192), (numel - 8 * 1000, 8 * 1000), (0, 4096)):
        want = oracle_sum(c_oracle, [a[lo:lo + n].cpu(), b[lo:lo + n].cpu()])
        assert_bit_equal(out[lo:lo + n], want, f"window at {lo}")
    del out
    gathered = tccl_amd.all_gather(a, 2)
    assert torch.equal(gathered[0].view(torch.int16), a.view(torch.int16))
    assert torch.equal(gathered[1].view(torch.int16), b.view(torch.int16))
    del gathered
    torch.cuda.empty_cache()
    d0 = torch.empty_like(a)
    d1 = torch.empty_like(a)
    rc = tccl_amd.load_library().tccl_tree_copy_step(b.data_ptr(), d0.data_ptr(), d1.data_ptr(), numel * 2, stream())
    assert rc == 0
    assert torch.equal(d0.view(torch.int16), b.view(torch.int16))
    assert torch.equal(d1.view(torch.int16), b.view(torch.int16))
    # in-place tree reduce step over the whole 4 GiB+ range: own <- 0 + child + own
    rc = tccl_amd.load_library().tccl_tree_reduce_step(d0.data_ptr(), a.data_ptr(), None, d0.data_ptr(), numel,
                                                       _lib.TCCL_BF16, stream())
    assert rc == 0
    for lo in range(0, numel, step):
        n = min(step, numel - lo)
        want = (a[lo:lo + n].float() + b[lo:lo + n].float()).to(torch.bfloat16)
        assert torch.equal(d0[lo:lo + n].view(torch.int16), want.view(torch.int16)), f"tree step slice at {lo}"


# ------------------------------------------------------------------ reduce-scatter

@pytest.mark.parametrize("world", [2, 4, 8])
@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform], ids=["bf16", "f32"])
def test_reduce_scatter_every_rank(world, maker, _gpu_hygiene, c_oracle):
    numel = 8 * world * 5_003
    bufs = maker(world, numel)
    g = upload(_gpu_hygiene, bufs)
    full = oracle_sum(c_oracle, bufs)
    per = numel // world
    ar = tccl_amd.one_shot_all_reduce(g.tensor(0))
    shares = []
    for r in range(world):
        got = tccl_amd.reduce_scatter(g.tensor(r))
        assert got.shape == (per,)
        assert_bit_equal(got, full[r * per:(r + 1) * per], f"rank {r}")
        assert_bit_equal(got, ar[r * per:(r + 1) * per], f"rank {r} vs all-reduce slice")
        shares.append(got)
    # all-gather of the shares is the all-reduce
    gs = tccl_amd.register(shares)
    _gpu_hygiene.append(gs)
    assert_bit_equal(tccl_amd.all_gather(shares[0], world).reshape(-1), ar, "AG o RS")


def test_reduce_scatter_config3(_gpu_hygiene, c_oracle):
    """Benchmark shape 3: W=8 inputs of 67,108,864 bf16 ~N(0,1), rank 3's 8,388,608-element
    share; then the same shapes in fp32 ~U(-1,1)."""
    world, numel, rank = 8, 67_108_864, 3
    per = numel // world
    for maker in (seeded_randn, seeded_uniform):
        bufs = maker(world, numel)
        g = upload(_gpu_hygiene, bufs)
        got = tccl_amd.reduce_scatter(g.tensor(rank))
        want = oracle_sum(c_oracle, [b[rank * per:(rank + 1) * per].contiguous() for b in bufs])
        assert_bit_equal(got, want, maker.__name__)
        tccl_amd.unregister(g)
        _gpu_hygiene.remove(g)
        del g, got, bufs
        gc.collect()
        torch.cuda.empty_cache()


def test_reduce_scatter_fill_rank(_gpu_hygiene):
    g = upload(_gpu_hygiene, [torch.full((8 * 8 * 64,), float(r), dtype=torch.bfloat16) for r in range(8)])
    for r in range(8):
        assert tccl_amd.reduce_scatter(g.tensor(r)).eq(28).all().item()


# ------------------------------------------------------------------ all-gather

@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform, seeded_int8], ids=["bf16", "f32", "int8"])
@pytest.mark.parametrize("numel", [16, 4096, 8_388_608])
def test_all_gather_equals_stack(maker, numel, _gpu_hygiene):
    """Benchmark shape 4 (numel = 8,388,608) and smaller; expected value as in
    triton_all_gather.py:128."""
    world = 8
    bufs = maker(world, numel)
    g = upload(_gpu_hygiene, bufs)
    out = tccl_amd.all_gather(g.tensor(2), world)
    assert out.shape == (world, numel) and out.dtype == bufs[0].dtype
    assert_bit_equal(out, torch.stack(bufs), maker.__name__)


def test_all_gather_fill_rank(_gpu_hygiene):
    """The reference's (commented) all-gather test, triton_all_gather.py:117-133: every rank
    fills 2,048 elements with its rank; the result is the stack of those."""
    world = 8
    g = upload(_gpu_hygiene, [torch.full((2048,), float(r), dtype=torch.bfloat16) for r in range(world)])
    want = torch.stack([torch.full((2048,), float(r), dtype=torch.bfloat16) for r in range(world)])
    for r in range(world):
        assert_bit_equal(tccl_amd.one_shot_all_gather(g.tensor(r), world), want, f"rank {r}")


@pytest.mark.parametrize("world", [1, 2, 3, 5, 8])
def test_all_gather_worlds_shapes_and_nan_payloads(world, _gpu_hygiene):
    rng = np.random.default_rng(world)
    bufs = [from_np_bits(rng.integers(0, 1 << 16, size=(24 * 8 * 11,), dtype=np.uint16)).reshape(24, 88)
            for _ in range(world)]                  # every bit pattern incl. NaN payloads
    g = upload(_gpu_hygiene, bufs)
    out = tccl_amd.one_shot_all_gather(g.tensor(0), world)
    assert out.shape == (world, 24, 88)
    assert_bit_equal(out, torch.stack(bufs), f"W={world}")


@pytest.mark.parametrize("unroll", [1, 2, 4])
@pytest.mark.parametrize("flags", [0, 3, 4])
def test_all_gather_launch_shapes(unroll, flags, _gpu_hygiene):
    bufs = seeded_int8(4, 16 * 70_001)
    g = upload(_gpu_hygiene, bufs)
    for block, tile_iters, grid in ((64, 0, 0), (256, 5, 16), (512, 1, 3)):
        cfg = tccl_amd.LaunchCfg(block=block, unroll=unroll, grid=grid, tile_iters=tile_iters, flags=flags)
        assert_bit_equal(tccl_amd.all_gather(g.tensor(0), 4, cfg=cfg), torch.stack(bufs), f"{block}/{unroll}")


@pytest.mark.parametrize("world", [2, 4, 8])
@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform], ids=["bf16", "f32"])
def test_two_shot_all_reduce_equals_one_shot(world, maker, _gpu_hygiene, c_oracle):
    numel = 8 * world * 20_011
    bufs = maker(world, numel)
    g = upload(_gpu_hygiene, bufs)
    want = oracle_sum(c_oracle, bufs)
    for r in (0, world - 1):
        assert_bit_equal(tccl_amd.two_shot_all_reduce(g.tensor(r)), want, f"two-shot rank {r}")
        assert_bit_equal(tccl_amd.all_reduce(g.tensor(r), "two_shot"), want, "by name")
    assert_bit_equal(tccl_amd.all_reduce(g.tensor(0)), want, "auto")
    with pytest.raises(ValueError):
        tccl_amd.all_reduce(g.tensor(0), "ring")


# ------------------------------------------------------------------ double-tree node steps

@pytest.mark.parametrize("children", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform], ids=["bf16", "f32"])
@pytest.mark.parametrize("in_place", [False, True])
def test_tree_reduce_step(children, maker, in_place, _gpu_hygiene, c_oracle):
    numel = 65_536 * 3 + 8 * 5                      # three 128 KiB chunks (bf16) and a bit
    own, c0, c1 = maker(3, numel, seed_base=40)
    k0 = c0 if children[0] else None
    k1 = c1 if children[1] else None
    want = torch_ref.tree_reduce_step(own, k0, k1)
    d_own, d0, d1 = own.to(DEV), c0.to(DEV), c1.to(DEV)
    dst = d_own if in_place else torch.empty_like(d_own)
    dt = _lib.TCCL_BF16 if own.dtype == torch.bfloat16 else _lib.TCCL_F32
    rc = tccl_amd.load_library().tccl_tree_reduce_step(
        d_own.data_ptr(), d0.data_ptr() if children[0] else None, d1.data_ptr() if children[1] else None,
        dst.data_ptr(), numel, dt, stream())
    assert rc == 0
    assert_bit_equal(dst, want, f"children={children}")
    assert_bit_equal(d0, c0, "child0 untouched")
    assert_bit_equal(d1, c1, "child1 untouched")


def test_tree_reduce_step_large_in_place(_gpu_hygiene, c_oracle):
    """128 MiB half of a 256 MiB bf16 buffer, own + two children, stored over own."""
    numel = 67_108_864
    torch.manual_seed(1)
    base = torch.randn(numel, dtype=torch.bfloat16)
    own, c0, c1 = base, base.roll(12_345_677), base.roll(-7_654_321)
    want = oracle_sum(c_oracle, [c0, c1, own])
    d_own, d0, d1 = own.to(DEV), c0.to(DEV), c1.to(DEV)
    rc = tccl_amd.load_library().tccl_tree_reduce_step(d_own.data_ptr(), d0.data_ptr(), d1.data_ptr(),
                                                       d_own.data_ptr(), numel, _lib.TCCL_BF16, stream())
    assert rc == 0
    assert_bit_equal(d_own, want, "in place, large")


@pytest.mark.parametrize("numel", [33_554_432, 33_554_432 + 8 * 1025 + 3], ids=["64MiB", "64MiB-ragged"])
def test_tree_reduce_step_two_children_in_place_full_tiles(numel, _gpu_hygiene, c_oracle):
    """64 MiB of output, own + two children, stored over own: the size at which three sources are cut
    into full 128 KiB tiles and take the kernel whose workgroup pairs share a region in alternate
    pieces -- each workgroup must have read all its pieces before it writes any.  Also with a ragged
    end (a partial tile and three elements beyond the last vector).  Children must come out untouched."""
    torch.manual_seed(7)
    base = torch.randn(numel, dtype=torch.bfloat16)
    own, c0, c1 = base, base.roll(9_876_543), base.roll(-3_456_789)
    want = oracle_sum(c_oracle, [c0, c1, own])
    d_own, d0, d1 = own.to(DEV), c0.to(DEV), c1.to(DEV)
    rc = tccl_amd.load_library().tccl_tree_reduce_step(d_own.data_ptr(), d0.data_ptr(), d1.data_ptr(),
                                                       d_own.data_ptr(), numel, _lib.TCCL_BF16, stream())
    assert rc == 0
    assert_bit_equal(d_own, want, "in place, full tiles")
    assert_bit_equal(d0, c0, "child0 untouched")
    assert_bit_equal(d1, c1, "child1 untouched")


@pytest.mark.parametrize("two", [False, True])
def test_tree_copy_step(two, _gpu_hygiene):
    src = seeded_int8(1, 16 * 100_003)[0]
    d_src = src.to(DEV)
    a = torch.zeros_like(d_src)
    b = torch.zeros_like(d_src)
    rc = tccl_amd.load_library().tccl_tree_copy_step(d_src.data_ptr(), a.data_ptr(), b.data_ptr() if two else None,
                                                     src.numel(), stream())
    assert rc == 0
    assert_bit_equal(a, src, "dst0")
    assert_bit_equal(b, src if two else torch.zeros_like(src), "dst1")


def test_tree_level_batch(_gpu_hygiene, c_oracle):
    """Several node steps of different kinds and lengths in one launch."""
    lib = tccl_amd.load_library()
    n1, n2 = 65_536 * 2 + 24, 8 * 777
    x = [t.to(DEV) for t in seeded_randn(6, n1, seed_base=60)]
    cpu = [t.cpu().clone() for t in x]
    outs = [torch.zeros(n1, dtype=torch.bfloat16, device=DEV) for _ in range(4)]
    jobs = (_lib.NodeJob * 4)()

    def fill(j, src, dst, numel, is_copy):
        for k in range(3):
            j.src[k] = src[k]
        for k in range(2):
            j.dst[k] = dst[k]
        j.numel, j.is_copy = numel, is_copy
    fill(jobs[0], [x[0].data_ptr(), x[1].data_ptr(), x[2].data_ptr()], [outs[0].data_ptr(), None], n1, 0)
    fill(jobs[1], [x[3].data_ptr(), None, x[4].data_ptr()], [x[4].data_ptr(), outs[1].data_ptr()], n2, 0)   # in place + 2nd dst
    fill(jobs[2], [x[5].data_ptr(), None, None], [outs[2].data_ptr(), outs[3].data_ptr()], n1, 1)
    # a leaf step in place on a buffer of its own (jobs of one launch must not share outputs)
    y = seeded_randn(1, n2, seed_base=99)[0]
    d_y = y.to(DEV)
    fill(jobs[3], [None, None, d_y.data_ptr()], [d_y.data_ptr(), None], n2, 0)
    for chunk in (0, 4096, 1 << 20):
        for o in outs:
            o.zero_()
        x[4].copy_(cpu[4])
        d_y.copy_(y)
        assert lib.tccl_tree_level(jobs, 4, _lib.TCCL_BF16, chunk, stream()) == 0
        assert_bit_equal(outs[0], torch_ref.tree_reduce_step(cpu[2], cpu[0], cpu[1]), "job 0")
        w1 = torch_ref.tree_reduce_step(cpu[4][:n2], cpu[3][:n2], None)
        assert_bit_equal(x[4][:n2], w1, "job 1 in place")
        assert_bit_equal(x[4][n2:], cpu[4][n2:], "job 1 beyond its range")
        assert_bit_equal(outs[1][:n2], w1, "job 1 second destination")
        assert_bit_equal(outs[2], cpu[5], "job 2 copy")
        assert_bit_equal(outs[3], cpu[5], "job 2 copy, second destination")
        assert_bit_equal(d_y, torch_ref.tree_reduce_step(y, None, None), "job 3")


# ------------------------------------------------------------------ full double tree

@pytest.mark.parametrize("world", [2, 4, 8, 16, 32])
@pytest.mark.parametrize("numel", [8, 16, 8 * 12_345, 65_536 * 4 + 8])
def test_double_tree_all_ranks(world, numel, _gpu_hygiene, c_oracle):
    bufs = seeded_randn(world, numel, seed_base=100)
    final, outs = c_oracle.double_tree_all_reduce_bf16([np_bits(b) for b in bufs])
    want = from_np_bits(outs[0])
    assert_bit_equal(want, torch_ref.double_tree_all_reduce(bufs)[0], "oracles agree")
    g = upload(_gpu_hygiene, bufs)
    got = [tccl_amd.double_tree_all_reduce(g.tensor(r), fused=False) for r in range(world)]   # one call per rank
    for r in range(world):
        assert_bit_equal(got[r], want, f"output of rank {r}")
        assert_bit_equal(g.tensor(r), from_np_bits(final[r]), f"buffer of rank {r}")


@pytest.mark.parametrize("world", [2, 4, 8])
@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform], ids=["bf16", "f32"])
@pytest.mark.parametrize("numel", [8, 24, 8 * 12_345, 65_536 * 4 + 8, 8 * 1_000_003])
def test_double_tree_one_launch_kernel(world, maker, numel, _gpu_hygiene, c_oracle):
    """The whole tree in one launch against the level schedule and the oracle: same outputs,
    same final buffers, bit for bit."""
    bufs = maker(world, numel, seed_base=300)
    want = torch_ref.double_tree_all_reduce(bufs)[0]
    if maker is seeded_randn:
        _, outs = c_oracle.double_tree_all_reduce_bf16([np_bits(b) for b in bufs])
        assert_bit_equal(from_np_bits(outs[0]), want, "oracles agree")
    g = upload(_gpu_hygiene, bufs)
    fused = tccl_amd.double_tree_all_reduce_world(g, fused=True)
    for r in range(world):
        assert_bit_equal(fused[r], want, f"one launch, output {r}")
        assert_bit_equal(g.tensor(r), want, f"one launch, buffer {r}")
    g2 = upload(_gpu_hygiene, bufs)
    levels = tccl_amd.double_tree_all_reduce_world(g2, fused=False)
    for r in range(world):
        assert_bit_equal(levels[r], fused[r], f"schedule vs one launch, output {r}")


def test_double_tree_one_launch_limits(_gpu_hygiene):
    g = tccl_amd.empty_world(16, 64, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    with pytest.raises(tccl_amd.TcclError):
        tccl_amd.double_tree_all_reduce_world(g, fused=True)          # worlds of 2, 4, 8 only
    assert len(tccl_amd.double_tree_all_reduce_world(g)) == 16         # auto falls back to the schedule
    lib = tccl_amd.load_library()
    assert lib.tccl_double_tree_all_reduce_fused(g.ptr_array, None, 3, 64, 0, None) == -3
    assert lib.tccl_double_tree_all_reduce_fused(g.ptr_array, None, 8, 60, 0, None) == -2


def test_double_tree_fill_rank_and_second_collective(_gpu_hygiene):
    world = 8
    g = upload(_gpu_hygiene, [torch.full((8192,), float(r), dtype=torch.bfloat16) for r in range(world)])
    for r in range(world):
        assert tccl_amd.double_tree_all_reduce(g.tensor(r)).eq(28).all().item()
    # every buffer now holds 28; the next collective sums those: 8 * 28
    for r in range(world):
        assert tccl_amd.double_tree_all_reduce(g.tensor(r)).eq(224).all().item()


@pytest.mark.parametrize("world,numel", [(8, 8 * 4099), (4, 65_536 * 3), (16, 8 * 513)])
def test_double_tree_plan_replays(world, numel, _gpu_hygiene, c_oracle):
    """The recorded plan against the eager schedule and the oracle, replayed several times
    with other work and synchronisations in between; every replay is checked."""
    g = tccl_amd.empty_world(world, numel, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    plan = tccl_amd.DoubleTreePlan(g)
    for rep in range(4):
        bufs = seeded_randn(world, numel, seed_base=1000 + 10 * rep)
        _, outs = c_oracle.double_tree_all_reduce_bf16([np_bits(b) for b in bufs])
        want = from_np_bits(outs[0])
        for r in range(world):
            g.tensor(r).copy_(bufs[r])
        got = plan.run()
        torch.cuda.synchronize()
        for r in range(world):
            assert_bit_equal(got[r], want, f"replay {rep} output {r}")
            assert_bit_equal(g.tensor(r), want, f"replay {rep} buffer {r}")
        # eager work between replays: the same collective without the plan
        for r in range(world):
            g.tensor(r).copy_(bufs[r])
        eager = tccl_amd.double_tree_all_reduce_world(g)
        assert_bit_equal(eager[0], want, f"eager after replay {rep}")
    plan.close()
    with pytest.raises(RuntimeError):
        plan.run()


def test_double_tree_f32_and_chunk_sizes(_gpu_hygiene, c_oracle):
    world, numel = 4, 4 * 50_001
    bufs = seeded_uniform(world, numel, seed_base=7)
    want = torch_ref.double_tree_all_reduce(bufs)[0]
    for chunk in (0, 1024, 1 << 22):
        g = upload(_gpu_hygiene, bufs)
        outs = tccl_amd.double_tree_all_reduce_world(g, chunk_elems=chunk)
        for r in range(world):
            assert_bit_equal(outs[r], want, f"chunk={chunk} rank {r}")


@pytest.mark.parametrize("how", ["level schedule", "default"])
def test_double_tree_config5_properties(how, _gpu_hygiene, c_oracle):
    """Benchmark shape 5: W=8 x 134,217,728 bf16 (256 MiB each), halves of
    67,108,864 elements, 65,536-element chunks.  Checked by size-independent properties:
    all 8 outputs and all 8 buffers are bit-identical, and windows of the result equal the
    oracle run on the same windows of the inputs.  Once with the level schedule and once with
    whatever the wrapper picks at this size (the pipelined single launch)."""
    world, numel = 8, 134_217_728
    torch.manual_seed(0)
    base = torch.randn(numel, dtype=torch.bfloat16)
    g = tccl_amd.empty_world(world, numel, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    shifts = [r * 7_000_001 for r in range(world)]
    dbase = base.to(DEV)
    for r in range(world):
        g.tensor(r).copy_(dbase.roll(shifts[r]))
    del dbase
    half = numel // 2
    windows = [(0, 65_536 * 2), (half - 65_536, 65_536), (half - 8, 8), (31_457_280, 8 * 1001)]
    samples = []
    for lo, n in windows:
        a = [g.tensor(r)[lo:lo + n].cpu() for r in range(world)]
        b = [g.tensor(r)[half + lo:half + lo + n].cpu() for r in range(world)]
        samples.append([torch.cat([x, y]) for x, y in zip(a, b)])
    if how == "level schedule":
        outs = tccl_amd.double_tree_all_reduce_world(g, chunk_elems=65_536, fused=False, pipelined=False)
    else:
        outs = tccl_amd.double_tree_all_reduce_world(g)
        assert tccl_amd.signal_pad_timeouts(g) == 0
    for r in range(1, world):
        assert torch.equal(outs[r].view(torch.int16), outs[0].view(torch.int16)), f"output {r}"
    for r in range(world):
        assert torch.equal(g.tensor(r).view(torch.int16), outs[0].view(torch.int16)), f"buffer {r}"
    for (lo, n), sample in zip(windows, samples):
        _, want = c_oracle.double_tree_all_reduce_bf16([np_bits(s) for s in sample])
        w = from_np_bits(want[0])
        assert_bit_equal(outs[0][lo:lo + n], w[:n], f"tree a window at {lo}")
        assert_bit_equal(outs[0][half + lo:half + lo + n], w[n:], f"tree b window at {lo}")


# ------------------------------------------------------------------ a client without Python

def test_plain_c_client():
    """tests/c_client/c_abi_client.c: hipMalloc'd buffers and the C entry points only (no
    torch anywhere in the process), built by `python -m tccl_amd.build`."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "c_client", "build", "c_abi_client")
    assert os.path.exists(exe), "C client not built: run `python -m tccl_amd.build`"
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = os.path.join(root, "tccl_amd") + os.pathsep + env.get("LD_LIBRARY_PATH", "")
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=120, env=env)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "c client ok" in proc.stdout


def test_probe_kernels_touch_what_they_say(_gpu_hygiene):
    """The measuring kernels: the read probe stores nothing (sources and sink unchanged, for
    every world and for ragged sizes), the write probe fills exactly the bytes it is given, the
    placement probe reports one record per workgroup."""
    from benchlib import probe
    lib = probe.load()
    for world, nbytes in [(1, 16), (3, 128 * 1024 + 48), (8, 5 * 128 * 1024 * 512 // 4 + 16), (8, 64 << 20)]:
        numel = nbytes // 2
        bufs = [torch.randn(numel, dtype=torch.float32, device=DEV).to(torch.bfloat16) for _ in range(world)]
        before = [b.clone() for b in bufs]
        sink = torch.zeros(4096, dtype=torch.uint8, device=DEV)
        ptrs = _lib.ptr_array([b.data_ptr() for b in bufs])
        assert lib.tccl_probe_read(ptrs, world, nbytes, sink.data_ptr(), stream()) == 0
        torch.cuda.synchronize()
        assert int(sink.count_nonzero().item()) == 0
        for b, want in zip(bufs, before):
            assert torch.equal(b.view(torch.int16), want.view(torch.int16))
    for nbytes in [16, 128 * 1024 - 16, 128 * 1024 * 513 + 32, 64 << 20]:
        guard = 256
        region = torch.full((nbytes + 2 * guard,), 0xAB, dtype=torch.uint8, device=DEV)
        for write in (lib.tccl_probe_write, lib.tccl_probe_write_small, lib.tccl_probe_write_dense):
            region.fill_(0xAB)
            assert write(region.data_ptr() + guard, nbytes, stream()) == 0
            torch.cuda.synchronize()
            assert bool((region[:guard] == 0xAB).all()) and bool((region[guard + nbytes:] == 0xAB).all())
            words = region[guard:guard + nbytes].view(torch.int32)
            assert bool((words[0::4] == 0x3F803F80).all()) and bool((words[3::4] == 0x3F803F80).all())
    assert lib.tccl_probe_empty(stream()) == 0
    where = torch.full((2 * 512,), -1, dtype=torch.int32, device=DEV)
    assert lib.tccl_probe_placement(where.data_ptr(), 512, 100, stream()) == 0
    torch.cuda.synchronize()
    xcd = where[1::2] & 15
    assert bool((where != -1).all()) and int(xcd.max()) <= 7
