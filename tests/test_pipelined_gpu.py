"""GPU parity of the pipelined double tree (one persistent launch, virtual ranks signalling
each other per chunk) against the CPU oracle and against the level schedule, through the C
ABI.  Bit-exact.  Every case also checks that no wait expired and that the signal pads are
zero-filled again afterwards."""
import ctypes
import gc

import pytest
import torch

import tccl_amd
from tccl_amd import _lib
from helpers import assert_bit_equal, from_np_bits, np_bits, seeded_randn, seeded_uniform
from oracle import torch_ref

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
# A wait that expires in the tests should do so quickly: 2^18 polls are some tenths of a second.
SPINS = 1 << 18


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
    g = tccl_amd.empty_world(len(bufs), bufs[0].shape, bufs[0].dtype, DEV)
    for r, b in enumerate(bufs):
        g.tensor(r).copy_(b)
    groups.append(g)
    return g


def cfg(workgroups=0, lag=0, spin_limit=SPINS, tile_kib=0, draw=False):
    """draw: the workgroups draw their places when they start to run (TCCL_PIPE_DRAW_PLACES)
    instead of taking them from their hardware index."""
    c = _lib.PipelineCfg(workgroups, lag, spin_limit, tile_kib)
    c.flags = _lib.PIPE_DRAW_PLACES if draw else 0
    return c


BINDINGS = pytest.mark.parametrize("draw", [False, True], ids=["by-index", "drawn"])


def pads_are_zero(group):
    return all(int(p.count_nonzero().item()) == 0 for p in group._signal_pads)   # noqa: SLF001


def run_and_check(group, want, what, **kw):
    print(f"pipelined: {what} {kw}", flush=True)
    outs = tccl_amd.double_tree_all_reduce_world(group, pipelined=True, **kw)
    chunk = kw.get("chunk_elems", 0)
    assert tccl_amd.signal_pad_timeouts(group) == 0, f"{what}: a wait expired"
    for r in range(group.world_size):
        assert_bit_equal(outs[r], want, f"{what}: output {r}")
        assert_bit_equal(group.tensor(r), want, f"{what}: buffer {r}")
    assert pads_are_zero(group), f"{what}: signal pads not reset"
    return outs


@pytest.mark.parametrize("world", [2, 4, 8])
@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform], ids=["bf16", "f32"])
@pytest.mark.parametrize("tile_kib", [32, 128])
@pytest.mark.parametrize("numel,chunk_elems", [
    (8, 0),                         # one vector: tree b only
    (16, 8),                        # one vector per tree, one-vector chunks
    (8 * 12_345, 0),                # one ragged chunk per tree
    (8 * 12_345, 512),              # hundreds of small chunks, last one ragged
    (65_536 * 6 + 8 * 77, 0),       # whole 128 KiB chunks plus a ragged one
    (8 * 1_000_003, 65_536 * 3),    # chunks larger than a tile
])
@BINDINGS
def test_pipelined_matches_oracle_and_schedule(world, maker, tile_kib, numel, chunk_elems, draw, _gpu_hygiene, c_oracle):
    bufs = maker(world, numel, seed_base=900)
    want = torch_ref.double_tree_all_reduce(bufs)[0]
    if maker is seeded_randn:
        _, outs = c_oracle.double_tree_all_reduce_bf16([np_bits(b) for b in bufs])
        assert_bit_equal(from_np_bits(outs[0]), want, "oracles agree")
    g = upload(_gpu_hygiene, bufs)
    got = run_and_check(g, want, f"W={world} n={numel} chunk={chunk_elems} tile={tile_kib} draw={draw}",
                        chunk_elems=chunk_elems, pipeline_cfg=cfg(tile_kib=tile_kib, draw=draw))
    g2 = upload(_gpu_hygiene, bufs)
    levels = tccl_amd.double_tree_all_reduce_world(g2, fused=False, chunk_elems=chunk_elems)
    for r in range(world):
        assert_bit_equal(levels[r], got[r], f"schedule vs pipelined, output {r}")


@pytest.mark.parametrize("tile_kib", [32, 128])
@pytest.mark.parametrize("workgroups,lag", [(8, 1), (8, 3), (16, 1), (64, 2), (256, 1), (256, 5), (0, 1), (0, 2), (0, 4)])
@BINDINGS
def test_pipelined_grid_and_lag(workgroups, lag, tile_kib, draw, _gpu_hygiene):
    """Any grid from one workgroup per rank upwards and any distance between the sweeps gives
    the same bits."""
    world, numel = 8, 65_536 * 40 + 4_096
    bufs = seeded_randn(world, numel, seed_base=910)
    want = torch_ref.double_tree_all_reduce(bufs)[0]
    g = upload(_gpu_hygiene, bufs)
    run_and_check(g, want, f"wgs={workgroups} lag={lag} tile={tile_kib} draw={draw}",
                  pipeline_cfg=cfg(workgroups, lag, tile_kib=tile_kib, draw=draw))


@BINDINGS
def test_pipelined_repeats_on_the_same_pads(draw, _gpu_hygiene):
    """The pads reset themselves: back-to-back collectives on one group, no clearing between."""
    world, numel = 8, 65_536 * 9
    g = tccl_amd.empty_world(world, numel, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    for round_ in range(4):
        bufs = seeded_randn(world, numel, seed_base=920 + 10 * round_)
        for r, b in enumerate(bufs):
            g.tensor(r).copy_(b)
        want = torch_ref.double_tree_all_reduce(bufs)[0]
        run_and_check(g, want, f"round {round_}", pipeline_cfg=cfg(draw=draw))


def test_pipelined_fill_rank(_gpu_hygiene):
    """The reference's self-test: every rank fills its buffer with its rank; all outputs are
    W(W-1)/2 (triton_one_shot_all_reduce_no_128.py:116-127)."""
    world = 8
    g = upload(_gpu_hygiene, [torch.full((65_536 * 4,), float(r), dtype=torch.bfloat16) for r in range(world)])
    outs = tccl_amd.double_tree_all_reduce_world(g, pipelined=True, pipeline_cfg=cfg())
    assert tccl_amd.signal_pad_timeouts(g) == 0
    for r in range(world):
        assert outs[r].eq(28).all().item()


def test_pipelined_without_outputs_through_c_abi(_gpu_hygiene):
    """outs = NULL: only the ranks' buffers receive the result."""
    world, numel = 4, 65_536 * 3 + 64
    bufs = seeded_randn(world, numel, seed_base=930)
    want = torch_ref.double_tree_all_reduce(bufs)[0]
    g = upload(_gpu_hygiene, bufs)
    lib = tccl_amd.load_library()
    need = lib.tccl_double_tree_signal_pad_bytes(world, numel, _lib.TCCL_BF16, 0)
    pads = g.signal_pads(need)
    c = cfg()
    s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.tccl_double_tree_all_reduce_pipelined(g.ptr_array, None, pads, g.signal_pad_bytes, world, numel,
                                                   _lib.TCCL_BF16, 0, ctypes.byref(c), s)
    assert rc == 0
    assert tccl_amd.signal_pad_timeouts(g) == 0
    for r in range(world):
        assert_bit_equal(g.tensor(r), want, f"buffer {r}")


@BINDINGS
def test_pipelined_full_size_properties(draw, _gpu_hygiene):
    """The full benchmark shape as the baseline words it (8 x 256 MiB bf16, pipelined in 128 KiB
    chunks = 65,536 elements, each worked as one 128 KiB tile): integer-valued inputs whose sum
    is exact in every order, so the expected result is known without a CPU pass.  Then once more
    with the library's own choice of chunk (32 KiB) on the same group."""
    world, numel = 8, 134_217_728
    g = tccl_amd.empty_world(world, numel, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    gen = torch.Generator(device=DEV).manual_seed(77)
    total = torch.zeros(numel, dtype=torch.float32, device=DEV)
    for r in range(world):
        vals = torch.randint(-8, 9, (numel,), generator=gen, device=DEV, dtype=torch.int32).to(torch.bfloat16)
        g.tensor(r).copy_(vals)
        total += vals.float()
    want = total.to(torch.bfloat16)       # |sum| <= 64: exact in bf16 at every node
    del total
    outs = tccl_amd.double_tree_all_reduce_world(g, pipelined=True, chunk_elems=65_536,
                                                 pipeline_cfg=cfg(spin_limit=1 << 20, tile_kib=128, draw=draw))
    assert tccl_amd.signal_pad_timeouts(g) == 0
    for r in range(world):
        assert torch.equal(outs[r], want), f"output {r}"
        assert torch.equal(g.tensor(r), want), f"buffer {r}"
    assert pads_are_zero(g)
    # the buffers now all hold `want`: their all-reduce is 8 * want, still exact (|sum| <= 512)
    outs = tccl_amd.double_tree_all_reduce_world(g, pipelined=True, pipeline_cfg=cfg(spin_limit=1 << 20, draw=draw))
    assert tccl_amd.signal_pad_timeouts(g) == 0
    want8 = (want.float() * 8).to(torch.bfloat16)
    for r in range(world):
        assert torch.equal(outs[r], want8), f"default chunks: output {r}"
        assert torch.equal(g.tensor(r), want8), f"default chunks: buffer {r}"
    assert pads_are_zero(g)


@BINDINGS
def test_pipelined_expired_waits_drain_and_recover(draw, _gpu_hygiene):
    """Failure handling, forced from the host: with a spin limit of one poll, waits expire (a
    parent polls before its children can have finished a chunk).  The launch must still end
    and count the time-outs, the next collective on the group must raise instead of working
    on half-reduced buffers, and after that the group must work again."""
    world, numel = 8, 65_536 * 64
    bufs = seeded_randn(world, numel, seed_base=940)
    want = torch_ref.double_tree_all_reduce(bufs)[0]
    g = upload(_gpu_hygiene, bufs)
    print("pipelined: spin limit 1", flush=True)
    tccl_amd.double_tree_all_reduce_world(g, pipelined=True, pipeline_cfg=cfg(spin_limit=1, draw=draw))
    torch.cuda.synchronize()                         # the grid drained
    expired = tccl_amd.signal_pad_timeouts(g)
    if expired == 0:                                 # every signal happened to be there already
        for r in range(world):
            assert_bit_equal(g.tensor(r), want, f"buffer {r}")
        return
    assert g.timeout_flag[0] == 1, "the kernel did not raise the host flag"
    with pytest.raises(tccl_amd.TcclError) as err:
        tccl_amd.double_tree_all_reduce_world(g, pipelined=True, pipeline_cfg=cfg(draw=draw))
    assert err.value.code == _lib.TCCL_ETIMEOUT
    assert g.timeout_flag[0] == 0 and pads_are_zero(g), "raising must leave the group usable"
    for r, b in enumerate(bufs):
        g.tensor(r).copy_(b)
    run_and_check(g, want, "after the error", pipeline_cfg=cfg(draw=draw))


def test_expired_wait_surfaces_at_the_next_collective_of_any_kind(_gpu_hygiene):
    """The per-rank wrappers never hand out results of a group whose last signalling launch
    timed out without saying so: whichever collective comes next raises (nobody has to know
    about signal_pad_timeouts), exactly once."""
    world, numel = 8, 65_536 * 64
    bufs = seeded_randn(world, numel, seed_base=945)
    g = upload(_gpu_hygiene, bufs)
    print("pipelined through the per-rank wrapper: spin limit 1", flush=True)
    tccl_amd.double_tree_all_reduce_world(g, pipelined=True, pipeline_cfg=cfg(spin_limit=1))
    torch.cuda.synchronize()
    if g.timeout_flag[0] == 0:
        pytest.skip("no wait happened to expire in this run")
    with pytest.raises(tccl_amd.TcclError, match="wait expired"):
        tccl_amd.one_shot_all_reduce(g.tensor(0))
    for r, b in enumerate(bufs):
        g.tensor(r).copy_(b)
    got = tccl_amd.one_shot_all_reduce(g.tensor(0))          # the error is reported once
    assert_bit_equal(got, torch_ref.all_reduce(bufs), "one-shot after the error")


def test_pipelined_argument_checks(_gpu_hygiene):
    lib = tccl_amd.load_library()
    g = tccl_amd.empty_world(16, 64, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    with pytest.raises(ValueError):
        tccl_amd.double_tree_all_reduce_world(g, pipelined=True)          # worlds of 2, 4, 8 only
    g8 = tccl_amd.empty_world(8, 64, torch.bfloat16, DEV)
    _gpu_hygiene.append(g8)
    need = lib.tccl_double_tree_signal_pad_bytes(8, 64, _lib.TCCL_BF16, 0)
    pads = g8.signal_pads(need)
    call = lib.tccl_double_tree_all_reduce_pipelined
    assert call(g8.ptr_array, None, pads, need - 16, 8, 64, _lib.TCCL_BF16, 0, None, None) == _lib.TCCL_EINVAL
    assert call(g8.ptr_array, None, None, need, 8, 64, _lib.TCCL_BF16, 0, None, None) == _lib.TCCL_EINVAL
    assert call(g8.ptr_array, None, pads, need, 8, 60, _lib.TCCL_BF16, 0, None, None) == _lib.TCCL_EALIGN
    assert call(g8.ptr_array, None, pads, need, 8, 64, _lib.TCCL_BF16, 12, None, None) == _lib.TCCL_EALIGN
    assert call(g8.ptr_array, None, pads, need, 3, 64, _lib.TCCL_BF16, 0, None, None) == _lib.TCCL_EPOW2
    assert call(g8.ptr_array, None, pads, need, 8, 0, _lib.TCCL_BF16, 0, None, None) == 0


# ---------------------------------------------------------------- one-launch two-shot all-reduce

def oracle_sum(c_oracle, bufs):
    if bufs[0].dtype == torch.bfloat16:
        return from_np_bits(c_oracle.all_reduce_bf16([np_bits(b) for b in bufs]))
    return torch.from_numpy(c_oracle.all_reduce_f32([b.numpy() for b in bufs]))


def two_shot_and_check(group, want, what, **kw):
    print(f"two-shot: {what} {kw}", flush=True)
    outs = tccl_amd.two_shot_all_reduce_world(group, **kw)
    assert tccl_amd.signal_pad_timeouts(group) == 0, f"{what}: a wait expired"
    for r in range(group.world_size):
        if outs is not None:
            assert_bit_equal(outs[r], want, f"{what}: output {r}")
        assert_bit_equal(group.tensor(r), want, f"{what}: buffer {r}")
    assert pads_are_zero(group), f"{what}: signal pads not reset"


@pytest.mark.parametrize("world", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("maker", [seeded_randn, seeded_uniform], ids=["bf16", "f32"])
@pytest.mark.parametrize("vecs_per_share", [1, 3, 1_023, 1_024, 1_025, 70_001])
@BINDINGS
def test_two_shot_one_launch_matches_oracle(world, maker, vecs_per_share, draw, _gpu_hygiene, c_oracle):
    """Every buffer and every output equals the one-shot all-reduce of the oracle, bit for
    bit: shares of one vector, around one 16 KiB tile (1,024 vectors) and many ragged tiles."""
    per_vec = 8 if maker is seeded_randn else 4
    numel = vecs_per_share * per_vec * world
    bufs = maker(world, numel, seed_base=950)
    want = oracle_sum(c_oracle, bufs)
    g = upload(_gpu_hygiene, bufs)
    two_shot_and_check(g, want, f"W={world} n={numel} draw={draw}", pipeline_cfg=cfg(draw=draw))
    one = tccl_amd.one_shot_all_reduce(upload(_gpu_hygiene, bufs).tensor(0))
    assert_bit_equal(one, want, "one-shot kernel agrees")


@pytest.mark.parametrize("workgroups", [8, 16, 24, 64, 512, 0])
@pytest.mark.parametrize("with_outputs", [True, False])
@BINDINGS
def test_two_shot_grid_and_in_place_only(workgroups, with_outputs, draw, _gpu_hygiene, c_oracle):
    world, numel = 8, 8 * 8 * 40_001
    bufs = seeded_randn(world, numel, seed_base=960)
    want = oracle_sum(c_oracle, bufs)
    g = upload(_gpu_hygiene, bufs)
    two_shot_and_check(g, want, f"wgs={workgroups} outs={with_outputs} draw={draw}", with_outputs=with_outputs,
                       pipeline_cfg=cfg(workgroups, draw=draw))


def test_two_shot_order_sensitive_and_repeats(_gpu_hygiene):
    """[2^24, 1 x 6, -2^24] sums to 0 only in rank order (fp32); then the same group again with
    fill(rank) -> 28, without clearing the pads."""
    world, numel = 8, 4 * 8 * 1_000
    vals = [2.0 ** 24, 1, 1, 1, 1, 1, 1, -(2.0 ** 24)]
    g = upload(_gpu_hygiene, [torch.full((numel,), v, dtype=torch.float32) for v in vals])
    two_shot_and_check(g, torch.zeros(numel, dtype=torch.float32), "rank order", pipeline_cfg=cfg())
    for r in range(world):
        g.tensor(r).fill_(float(r))
    two_shot_and_check(g, torch.full((numel,), 28.0, dtype=torch.float32), "fill(rank)", pipeline_cfg=cfg())


@BINDINGS
def test_two_shot_full_size(draw, _gpu_hygiene):
    """The headline shape, 8 x 64 MiB bf16: against the one-shot kernel's result."""
    world, numel = 8, 33_554_432
    g = tccl_amd.empty_world(world, numel, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    gen = torch.Generator(device=DEV).manual_seed(5)
    for r in range(world):
        g.tensor(r).copy_(torch.randn(numel, generator=gen, device=DEV, dtype=torch.float32))
    want = tccl_amd.one_shot_all_reduce(g.tensor(0))
    outs = tccl_amd.two_shot_all_reduce_world(g, pipeline_cfg=cfg(spin_limit=1 << 20, draw=draw))
    assert tccl_amd.signal_pad_timeouts(g) == 0
    for r in range(world):
        assert torch.equal(outs[r].view(torch.int16), want.view(torch.int16)), f"output {r}"
        assert torch.equal(g.tensor(r).view(torch.int16), want.view(torch.int16)), f"buffer {r}"
    assert pads_are_zero(g)


@BINDINGS
def test_two_shot_expired_barrier_drains_and_recovers(draw, _gpu_hygiene, c_oracle):
    """Failure handling, forced from the host: with one poll per wait the barrier expires
    unless every peer happens to be there already; the launch ends either way, the next
    collective raises, and then the group works again."""
    world, numel = 8, 8 * 8 * 200_000
    bufs = seeded_randn(world, numel, seed_base=970)
    want = oracle_sum(c_oracle, bufs)
    g = upload(_gpu_hygiene, bufs)
    print("two-shot: spin limit 1", flush=True)
    tccl_amd.two_shot_all_reduce_world(g, pipeline_cfg=cfg(spin_limit=1, draw=draw))
    torch.cuda.synchronize()
    if tccl_amd.signal_pad_timeouts(g) == 0:
        for r in range(world):
            assert_bit_equal(g.tensor(r), want, f"buffer {r}")
        return
    assert g.timeout_flag[0] == 1, "the kernel did not raise the host flag"
    with pytest.raises(tccl_amd.TcclError) as err:
        tccl_amd.two_shot_all_reduce_world(g, pipeline_cfg=cfg())
    assert err.value.code == _lib.TCCL_ETIMEOUT
    for r, b in enumerate(bufs):
        g.tensor(r).copy_(b)
    two_shot_and_check(g, want, "after the error", pipeline_cfg=cfg())


def test_two_shot_argument_checks(_gpu_hygiene):
    lib = tccl_amd.load_library()
    g = tccl_amd.empty_world(8, 8 * 8 * 4, torch.bfloat16, DEV)
    _gpu_hygiene.append(g)
    pads = g.signal_pads(4096)
    call = lib.tccl_two_shot_all_reduce
    assert call(g.ptr_array, None, pads, 4096, 9, 256, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL
    assert call(g.ptr_array, None, pads, 16, 8, 256, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL   # pad too small
    assert call(g.ptr_array, None, None, 4096, 8, 256, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL
    assert call(g.ptr_array, None, pads, 4096, 8, 8 * 9, _lib.TCCL_BF16, None, None) == _lib.TCCL_EALIGN
    assert call(g.ptr_array, None, pads, 4096, 8, 256, 7, None, None) == _lib.TCCL_EINVAL
    assert call(g.ptr_array, None, pads, 4096, 8, 0, _lib.TCCL_BF16, None, None) == 0


def test_signalling_kernels_on_two_streams_are_kept_apart(_gpu_hygiene, c_oracle):
    """Two signalling kernels at once could starve each other of workgroup slots; the library
    chains them with an event, so launching a pipelined tree and a two-shot all-reduce on two
    different streams back to back, several times, still gives exact results and no expired
    wait."""
    world, numel = 8, 65_536 * 48
    bufs_a = seeded_randn(world, numel, seed_base=980)
    bufs_b = seeded_randn(world, numel, seed_base=990)
    want_a = torch_ref.double_tree_all_reduce(bufs_a)[0]
    want_b = oracle_sum(c_oracle, bufs_b)
    ga, gb = upload(_gpu_hygiene, bufs_a), upload(_gpu_hygiene, bufs_b)
    ga.signal_pads(1 << 16)
    gb.signal_pads(1 << 16)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    for round_ in range(3):
        print(f"two streams: round {round_}", flush=True)
        for r in range(world):
            ga.tensor(r).copy_(bufs_a[r])
            gb.tensor(r).copy_(bufs_b[r])
        torch.cuda.synchronize()
        with torch.cuda.stream(s1):
            outs_a = tccl_amd.double_tree_all_reduce_world(ga, pipelined=True, pipeline_cfg=cfg())
        with torch.cuda.stream(s2):
            tccl_amd.two_shot_all_reduce_world(gb, with_outputs=False, pipeline_cfg=cfg())
        torch.cuda.synchronize()
        assert tccl_amd.signal_pad_timeouts(ga) == 0 and tccl_amd.signal_pad_timeouts(gb) == 0
        for r in range(world):
            assert_bit_equal(outs_a[r], want_a, f"tree output {r}")
            assert_bit_equal(gb.tensor(r), want_b, f"two-shot buffer {r}")


def test_signalling_kernels_can_be_captured_in_a_graph(_gpu_hygiene, c_oracle):
    """Both signalling entry points recorded into a caller's HIP graph (through
    torch.cuda.graph), replayed several times with new inputs and an eager signalling call in
    between; every replay is checked, and the pads are clean after each."""
    world, numel = 8, 65_536 * 20 + 8 * 8 * 33
    lib = tccl_amd.load_library()
    ga = tccl_amd.empty_world(world, numel, torch.bfloat16, DEV)
    gb = tccl_amd.empty_world(world, numel, torch.bfloat16, DEV)
    _gpu_hygiene.extend([ga, gb])
    need = lib.tccl_double_tree_signal_pad_bytes(world, numel, _lib.TCCL_BF16, 0)
    pads_a, pads_b = ga.signal_pads(max(need, 1 << 15)), gb.signal_pads(1 << 15)
    outs = torch.empty((world, numel), dtype=torch.bfloat16, device=DEV)
    out_ptrs = _lib.ptr_array([int(outs[r].data_ptr()) for r in range(world)])
    c = cfg()

    def enqueue():
        s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert lib.tccl_double_tree_all_reduce_pipelined(ga.ptr_array, out_ptrs, pads_a, ga.signal_pad_bytes, world,
                                                         numel, _lib.TCCL_BF16, 0, ctypes.byref(c), s) == 0
        assert lib.tccl_two_shot_all_reduce(gb.ptr_array, None, pads_b, gb.signal_pad_bytes, world, numel,
                                            _lib.TCCL_BF16, ctypes.byref(c), s) == 0

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue()                                  # warm-up outside the capture (first-use queries happen here)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    for rep in range(3):
        print(f"captured signalling kernels: replay {rep}", flush=True)
        bufs = seeded_randn(world, numel, seed_base=1000 + 10 * rep)
        for r in range(world):
            ga.tensor(r).copy_(bufs[r])
            gb.tensor(r).copy_(bufs[r])
        outs.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert tccl_amd.signal_pad_timeouts(ga) == 0 and tccl_amd.signal_pad_timeouts(gb) == 0
        tree_want = torch_ref.double_tree_all_reduce(bufs)[0]
        flat_want = oracle_sum(c_oracle, bufs)
        for r in range(world):
            assert_bit_equal(outs[r], tree_want, f"replay {rep}: tree output {r}")
            assert_bit_equal(gb.tensor(r), flat_want, f"replay {rep}: two-shot buffer {r}")
        assert pads_are_zero(ga) and pads_are_zero(gb)
        # an eager signalling call between replays
        for r in range(world):
            gb.tensor(r).copy_(bufs[r])
        two_shot_and_check(gb, flat_want, f"eager after replay {rep}", with_outputs=False, pipeline_cfg=cfg())
