"""The entry point that allocates nothing: tccl_two_shot_all_reduce_static keeps its signal
pads in a static device array inside the library.  Called through the C ABI and compared,
bit for bit, with tccl_two_shot_all_reduce (caller-owned pads) and with the C oracle on the same
inputs: two calls in a row, the second on a smaller input, then after a call whose waits were
made to expire from the host (the array must not carry that call's flags over), and recorded
into a HIP graph that is replayed with new inputs."""
import ctypes
import gc

import pytest
import torch

import tccl_amd
from tccl_amd import _lib
from helpers import assert_bit_equal, from_np_bits, np_bits, seeded_randn, seeded_uniform

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
SPINS = 1 << 18


@pytest.fixture(autouse=True)
def _gpu_hygiene():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    tccl_amd.load_library()
    yield
    torch.cuda.synchronize()
    gc.collect()
    torch.cuda.empty_cache()


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def oracle_sum(c_oracle, bufs):
    if bufs[0].dtype == torch.bfloat16:
        return from_np_bits(c_oracle.all_reduce_bf16([np_bits(b) for b in bufs]))
    return torch.from_numpy(c_oracle.all_reduce_f32([b.numpy() for b in bufs]))


def with_caller_pads(lib, bufs_host, numel, dtype_code, want_outputs):
    """The existing entry point: fresh device copies, fresh zeroed pads."""
    world = len(bufs_host)
    bufs = [b[:numel].to(DEV) for b in bufs_host]
    outs = [torch.empty_like(b) for b in bufs] if want_outputs else None
    pads = [torch.zeros(4 * (8 * 1024 + 288), dtype=torch.uint8, device=DEV) for _ in range(world)]
    cfg = _lib.PipelineCfg(0, 0, SPINS, 0)
    rc = lib.tccl_two_shot_all_reduce(
        _lib.ptr_array([b.data_ptr() for b in bufs]), _lib.ptr_array([o.data_ptr() for o in outs]) if outs else None,
        _lib.ptr_array([p.data_ptr() for p in pads]), pads[0].numel(), world, numel, dtype_code, ctypes.byref(cfg),
        stream())
    assert rc == 0
    torch.cuda.synchronize()
    n = ctypes.c_uint(0)
    assert lib.tccl_signal_pad_timeouts(pads[0].data_ptr(), pads[0].numel(), ctypes.byref(n), stream()) == 0
    assert n.value == 0
    return bufs, outs


def with_static_pads(lib, bufs_host, numel, dtype_code, want_outputs, spin_limit=SPINS, flag=None, draw=False):
    world = len(bufs_host)
    bufs = [b[:numel].to(DEV) for b in bufs_host]
    outs = [torch.empty_like(b) for b in bufs] if want_outputs else None
    cfg = _lib.PipelineCfg(0, 0, spin_limit, 0)
    cfg.flags = _lib.PIPE_DRAW_PLACES if draw else 0
    if flag is not None:
        cfg.timeout_flag = flag
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
    free_before, _ = torch.cuda.mem_get_info(DEV)
    rc = lib.tccl_two_shot_all_reduce_static(
        _lib.ptr_array([b.data_ptr() for b in bufs]), _lib.ptr_array([o.data_ptr() for o in outs]) if outs else None,
        world, numel, dtype_code, ctypes.byref(cfg), stream())
    assert rc == 0
    assert torch.cuda.memory_stats(DEV)["allocation.all.allocated"] == before     # nothing went through torch ...
    assert torch.cuda.mem_get_info(DEV)[0] == free_before                         # ... and no hipMalloc behind torch's back
    torch.cuda.synchronize()
    return bufs, outs


@pytest.mark.parametrize("maker,code", [(seeded_randn, _lib.TCCL_BF16), (seeded_uniform, _lib.TCCL_F32)],
                         ids=["bf16", "f32"])
@pytest.mark.parametrize("world", [8, 3])
@pytest.mark.parametrize("draw", [False, True], ids=["by-index", "drawn"])
def test_static_pads_two_calls_in_a_row_second_smaller(maker, code, world, draw, c_oracle):
    lib = tccl_amd.load_library()
    per_vec = 8 if code == _lib.TCCL_BF16 else 4
    big = per_vec * world * 70_001          # many ragged tiles per share
    small = per_vec * world * 1_025         # a little more than one tile per share
    host = maker(world, big, seed_base=1200)
    flag = ctypes.POINTER(ctypes.c_uint32)()
    assert lib.tccl_timeout_flag_create(ctypes.byref(flag)) == 0
    try:
        for what, numel, outputs in (("first call", big, True), ("second call, smaller", small, True),
                                     ("third call, in place only", big, False)):
            print(f"static pads: W={world} {what} numel={numel}", flush=True)
            want_bufs, want_outs = with_caller_pads(lib, host, numel, code, outputs)
            got_bufs, got_outs = with_static_pads(lib, host, numel, code, outputs, flag=flag, draw=draw)
            assert flag[0] == 0, f"{what}: a wait expired"
            want = oracle_sum(c_oracle, [b[:numel] for b in host])
            for r in range(world):
                assert_bit_equal(got_bufs[r], want_bufs[r], f"{what}: buffer {r}")
                assert_bit_equal(got_bufs[r], want, f"{what}: buffer {r} against the oracle")
                if outputs:
                    assert_bit_equal(got_outs[r], want_outs[r], f"{what}: output {r}")
                    assert_bit_equal(got_outs[r], want, f"{what}: output {r} against the oracle")
    finally:
        assert lib.tccl_timeout_flag_destroy(flag) == 0


def test_static_pads_are_clean_after_a_call_whose_waits_expired():
    """One poll per wait makes the barrier expire (unless every peer happens to be there):
    that call leaves raised flags behind in the array.  The next call must not see them."""
    lib = tccl_amd.load_library()
    world, numel = 8, 8 * 8 * 200_000
    host = seeded_randn(world, numel, seed_base=1210)
    flag = ctypes.POINTER(ctypes.c_uint32)()
    assert lib.tccl_timeout_flag_create(ctypes.byref(flag)) == 0
    try:
        print("static pads: spin limit 1", flush=True)
        with_static_pads(lib, host, numel, _lib.TCCL_BF16, False, spin_limit=1, flag=flag)
        print(f"static pads: host flag after the forced call = {flag[0]}", flush=True)
        flag[0] = 0
        want_bufs, _ = with_caller_pads(lib, host, numel, _lib.TCCL_BF16, False)
        for round_ in range(2):
            got_bufs, _ = with_static_pads(lib, host, numel, _lib.TCCL_BF16, False, flag=flag)
            assert flag[0] == 0
            for r in range(world):
                assert_bit_equal(got_bufs[r], want_bufs[r], f"round {round_}: buffer {r}")
    finally:
        assert lib.tccl_timeout_flag_destroy(flag) == 0


def test_static_pads_recorded_into_a_graph_and_replayed(c_oracle):
    """What the entry point is for: after one call outside (the one-time set-up: the array's address, the
    library's event), the call is captured into a HIP graph and replayed with new inputs; between the
    replays the program does eager work and synchronises.  Every replay against the oracle."""
    lib = tccl_amd.load_library()
    world, numel = 8, 8 * 8 * 30_011
    bufs = [torch.zeros(numel, dtype=torch.bfloat16, device=DEV) for _ in range(world)]
    outs = [torch.zeros(numel, dtype=torch.bfloat16, device=DEV) for _ in range(world)]
    bptr, optr = _lib.ptr_array([b.data_ptr() for b in bufs]), _lib.ptr_array([o.data_ptr() for o in outs])
    flag = ctypes.POINTER(ctypes.c_uint32)()
    assert lib.tccl_timeout_flag_create(ctypes.byref(flag)) == 0
    cfg = _lib.PipelineCfg(0, 0, SPINS, 0)
    cfg.timeout_flag = flag
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                       # warm-up outside the capture
            assert lib.tccl_two_shot_all_reduce_static(bptr, optr, world, numel, _lib.TCCL_BF16, ctypes.byref(cfg), stream()) == 0
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            assert lib.tccl_two_shot_all_reduce_static(bptr, optr, world, numel, _lib.TCCL_BF16, ctypes.byref(cfg), stream()) == 0
        for rep in range(3):
            host = seeded_randn(world, numel, seed_base=1300 + 10 * rep)
            for r in range(world):
                bufs[r].copy_(host[r])
                outs[r].zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert flag[0] == 0, f"replay {rep}: a wait expired"
            want = oracle_sum(c_oracle, host)
            for r in range(world):
                assert_bit_equal(outs[r], want, f"replay {rep}: output {r}")
                assert_bit_equal(bufs[r], want, f"replay {rep}: buffer {r}")
            (bufs[0].float().sum() + 1).item()              # eager work and a synchronisation between replays
        del graph
    finally:
        assert lib.tccl_timeout_flag_destroy(flag) == 0


def test_static_pads_limits_and_argument_checks():
    lib = tccl_amd.load_library()
    world, numel = 8, 8 * 8 * 16
    bufs = [torch.zeros(numel, dtype=torch.bfloat16, device=DEV) for _ in range(world)]
    ptrs = _lib.ptr_array([b.data_ptr() for b in bufs])
    call = lib.tccl_two_shot_all_reduce_static
    too_many = _lib.PipelineCfg(1024 * world + 1, 0, SPINS, 0)
    assert call(ptrs, None, world, numel, _lib.TCCL_BF16, ctypes.byref(too_many), stream()) == _lib.TCCL_ESCRATCH
    assert b"scratch" in lib.tccl_error_string(_lib.TCCL_ESCRATCH)
    assert call(ptrs, None, 9, numel, _lib.TCCL_BF16, None, stream()) == _lib.TCCL_EINVAL
    assert call(ptrs, None, world, numel + 8, _lib.TCCL_BF16, None, stream()) == _lib.TCCL_EALIGN
    assert call(None, None, world, numel, _lib.TCCL_BF16, None, stream()) == _lib.TCCL_EINVAL
    assert call(ptrs, None, world, 0, _lib.TCCL_BF16, None, stream()) == 0
    most = _lib.PipelineCfg(1024 * world, 0, SPINS, 0)          # the most the array has flags for: clamped to what fits
    assert call(ptrs, None, world, numel, _lib.TCCL_BF16, ctypes.byref(most), stream()) == 0
    torch.cuda.synchronize()
