#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the one the headline metric is quoted on): one-shot all-reduce (sum) over W=8
virtual-rank buffers of 64 MiB bf16 each (33,554,432 elements ~N(0,1), seeded per rank),
all resident in HBM before the timed region.  A step is one call of
``tccl_amd.one_shot_all_reduce`` (output allocation from torch's caching allocator plus one
kernel launch through the C ABI).  Prints ONE JSON line on stdout.

Algorithmic bytes per step: (W + 1) * N * 2 = 603,979,776 (W*N read, N written).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published
WORLD = 8
BYTES_PER_BUF = 64 << 20
LAT_BYTES_PER_BUF = 1 << 20

# HBM bytes per launch of the headline kernel from two rocprofv3 --pmc runs of this script
# (FETCH_SIZE 262,354.07 KiB and WRITE_SIZE 65,536.00 KiB per dispatch), each scaled by what
# the same counter reads for the 256 MiB plain copy of --calibrate-copy (factors 1.99959 and
# 0.99996): 524,600 KiB fetched + 65,533 KiB written.
MEASURED_TRAFFIC_BYTES = 604_296_372


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=150,
                   help="untimed steps first; 150 (13 ms) because launches 30-100 after idle run 1-2 %% slower "
                        "than the steady state while the clocks settle")
    p.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timing")
    p.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU work budget for the baseline leg")
    p.add_argument("--no-other-ops", action="store_true",
                   help="skip the short timings of reduce-scatter, all-gather and the tree node steps")
    p.add_argument("--calibrate-copy", action="store_true",
                   help="also run 20 plain copies of 256 MiB (tccl_tree_copy_step), so that a rocprofv3 --pmc "
                        "run of this command holds a kernel of known traffic to scale the counters by")
    p.add_argument("--sweep", action="store_true",
                   help="also time every op and size of the sweep; written to stderr as JSON lines")
    return p.parse_args()


class HipEvents:
    """HIP events from the library, recorded on the stream the kernels are launched on."""

    def __init__(self, lib, n):
        self.lib = lib
        self.ev = []
        for _ in range(n):
            e = ctypes.c_void_p()
            assert lib.tccl_event_create(ctypes.byref(e)) == 0
            self.ev.append(e)

    def record(self, i, stream):
        assert self.lib.tccl_event_record(self.ev[i], stream) == 0

    def elapsed_ms(self, i, j):
        assert self.lib.tccl_event_synchronize(self.ev[j]) == 0
        ms = ctypes.c_float()
        assert self.lib.tccl_event_elapsed_ms(self.ev[i], self.ev[j], ctypes.byref(ms)) == 0
        return float(ms.value)

    def close(self):
        for e in self.ev:
            self.lib.tccl_event_destroy(e)


def make_world(tccl_amd, torch, world, numel, dtype, device):
    group = tccl_amd.empty_world(world, numel, dtype, device)
    for r in range(world):
        gen = torch.Generator(device=device)
        gen.manual_seed(r)
        if dtype == torch.int8:
            group.tensor(r).copy_(torch.randint(-128, 128, (numel,), dtype=dtype, device=device, generator=gen))
        else:
            group.tensor(r).copy_(torch.randn(numel, dtype=torch.float32, device=device, generator=gen))
    return group


def time_steps(torch, lib, fn, steps, warmup):
    """(wall ms per step, HIP-event ms per step) over exactly `steps` calls."""
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev = HipEvents(lib, 2)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev.record(0, stream)
    for _ in range(steps):
        fn()
    ev.record(1, stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    dev_ms = ev.elapsed_ms(0, 1) / steps
    ev.close()
    return wall_ms, dev_ms


def latency_p50_us(torch, lib, fn, reps=300, warmup=30):
    """Median over single-launch HIP-event pairs."""
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev = HipEvents(lib, 2 * reps)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    for i in range(reps):
        ev.record(2 * i, stream)
        fn()
        ev.record(2 * i + 1, stream)
    torch.cuda.synchronize()
    us = sorted(ev.elapsed_ms(2 * i, 2 * i + 1) * 1e3 for i in range(reps))
    ev.close()
    return statistics.median(us), us[int(0.99 * (reps - 1))]


def cpu_baseline(torch, bufs_cpu, seconds):
    """The torch CPU oracle on the same workload, all host cores torch will use."""
    from oracle import torch_ref
    acc = torch.zeros(bufs_cpu[0].shape, dtype=torch.float32)
    times = []
    torch_ref.all_reduce(bufs_cpu, acc)                      # warm-up
    t_end = time.perf_counter() + seconds
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 50):
        t0 = time.perf_counter()
        torch_ref.all_reduce(bufs_cpu, acc)
        times.append(time.perf_counter() - t0)
    return statistics.median(times), len(times)


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: W virtual ranks are W buffers on the same MI355X; "
              "runs with --gpus above 1 are not part of this build", file=sys.stderr)
        sys.exit(2)

    import torch
    import tccl_amd
    lib = tccl_amd.load_library()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    device = "cuda:0"
    torch.cuda.set_device(0)

    numel = BYTES_PER_BUF // 2
    group = make_world(tccl_amd, torch, WORLD, numel, torch.bfloat16, device)
    mine = group.tensor(0)
    algo_bytes = (WORLD + 1) * numel * 2

    def step():
        return tccl_amd.one_shot_all_reduce(mine)

    wall_ms, dev_ms = time_steps(torch, lib, step, args.steps, args.warmup)
    gbs_wall = algo_bytes / (wall_ms * 1e-3) / 1e9
    gbs_dev = algo_bytes / (dev_ms * 1e-3) / 1e9

    # The same step rotated over 8 disjoint sets of inputs AND outputs (4.6 GiB touched between
    # two uses of any byte).  On one set the 256 MB memory-side cache absorbs the 64 MiB of
    # output writes (the same output lines are rewritten every step before they are evicted)
    # and serves a little of the input; rotated like this every byte really moves over HBM.
    rot_ms = None
    try:
        extra = [make_world(tccl_amd, torch, WORLD, numel, torch.bfloat16, device) for _ in range(7)]
        firsts = [mine] + [g.tensor(0) for g in extra]
        outs = [torch.empty_like(mine) for _ in range(8)]
        turn = [0]

        def rotated_step():
            turn[0] += 1
            return tccl_amd.one_shot_all_reduce(firsts[turn[0] % 8], out=outs[turn[0] % 8])

        _, rot_ms = time_steps(torch, lib, rotated_step, args.steps, args.warmup)
        for g in extra:
            tccl_amd.unregister(g)
        del extra, firsts, outs
    except RuntimeError as e:            # e.g. not enough free memory for seven more sets
        print(f"rotated measurement skipped: {e}", file=sys.stderr)

    # What the memory system gives the two halves of that launch on their own: a pure read pass
    # over the same 8 buffers and a pure write pass over one output, same launch shape.  The sum
    # is a read phase followed by a write burst, so their total is its practical bound here.
    sink = torch.zeros(4096, dtype=torch.uint8, device=device)
    probe_out = torch.empty_like(mine)
    pstream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _, read_ms = time_steps(torch, lib, lambda: lib.tccl_probe_read(group.ptr_array, WORLD, BYTES_PER_BUF,
                                                                    sink.data_ptr(), pstream), 100, 50)
    _, write_ms = time_steps(torch, lib, lambda: lib.tccl_probe_write(probe_out.data_ptr(), BYTES_PER_BUF, pstream),
                             100, 50)
    ceilings = {
        "read_8x64MiB_us": round(read_ms * 1e3, 2), "read_gbs": round(WORLD * BYTES_PER_BUF / (read_ms * 1e-3) / 1e9, 1),
        "write_64MiB_us": round(write_ms * 1e3, 2), "write_gbs": round(BYTES_PER_BUF / (write_ms * 1e-3) / 1e9, 1),
        "read_pass_plus_write_pass_us": round((read_ms + write_ms) * 1e3, 2),
        "sum_kernel_us": round(dev_ms * 1e3, 2),
        "note": "tccl_probe_read / tccl_probe_write: the read half and the write half of the sum kernel on their "
                "own, same buffers and launch shape, 100 launches each",
    }
    del probe_out

    # p50 latency at 1 MiB per buffer: prefix views of the same allocations
    lat_numel = LAT_BYTES_PER_BUF // 2
    small = mine[:lat_numel]
    p50_us, p99_us = latency_p50_us(torch, lib, lambda: tccl_amd.one_shot_all_reduce(small))
    # the same launch through the C entry point alone (output allocated once, no wrapper work)
    small_out = torch.empty_like(small)
    raw_stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    c_call = lambda: lib.tccl_all_reduce_sum(group.ptr_array, WORLD, small_out.data_ptr(), lat_numel, 0, raw_stream)
    p50_c_us, _ = latency_p50_us(torch, lib, c_call)
    # and what one wrapper call costs end to end when calls are issued back to back
    back_wall_ms, back_dev_ms = time_steps(torch, lib, lambda: tccl_amd.one_shot_all_reduce(small), 500, 50)

    cu = ctypes.c_int()
    clk = ctypes.c_int()
    bus = ctypes.c_int()
    l2 = ctypes.c_size_t()
    lib.tccl_device_info(ctypes.byref(cu), ctypes.byref(clk), ctypes.byref(bus), ctypes.byref(l2))

    result = {
        "metric": "achieved HBM GB/s (% of 8 TB/s) W=8 bf16 reduce @64MiB/buf; p50 us @1MiB",
        "value": round(gbs_wall, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",                      # the sums are accumulated in fp32 ...
        "io_dtype": "bf16",                  # ... over bf16 inputs, rounded once to a bf16 output
        "data": "synthetic N(0,1), seeded per virtual rank, resident in HBM",
        "config": {"workload": "one-shot all-reduce sum, W=8 virtual ranks, 64 MiB bf16 per buffer "
                               "(33,554,432 elements), one MI355X",
                   "world": WORLD, "bytes_per_buffer": BYTES_PER_BUF, "algorithmic_bytes_per_step": algo_bytes},
        "pct_of_peak": round(100.0 * gbs_wall / HBM_PEAK_GBS, 2),
        "rotated_over_8_buffer_sets": None if rot_ms is None else {
            "gbs": round(algo_bytes / (rot_ms * 1e-3) / 1e9, 1), "avg_launch_us": round(rot_ms * 1e3, 2)},
        "memory_system_ceilings": ceilings,
        "p50_us_at_1MiB": round(p50_us, 2),
        "p99_us_at_1MiB": round(p99_us, 2),
        "p50_us_at_1MiB_c_entry_point_only": round(p50_c_us, 2),
        "us_per_call_at_1MiB_back_to_back": round(back_dev_ms * 1e3, 2),
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbs_dev, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs_dev / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES,
            "kernel": "tccl::sum_phased_kernel<Bf16Sum, 8, 1, true>",
            "avg_launch_us": round(dev_ms * 1e3, 2),
            "algorithmic_bytes": algo_bytes,
        },
        "device": {"name": torch.cuda.get_device_name(0), "compute_units": cu.value,
                   "mem_clock_khz": clk.value, "mem_bus_bits": bus.value, "l2_bytes": l2.value},
    }

    if not args.no_cpu_baseline:
        bufs_cpu = [group.tensor(r).cpu() for r in range(WORLD)]
        med_s, nruns = cpu_baseline(torch, bufs_cpu, args.cpu_seconds)
        # the GPU result must equal the CPU oracle's on the very same inputs
        from oracle import torch_ref
        same = torch.equal(step().cpu().view(torch.int16), torch_ref.all_reduce(bufs_cpu).view(torch.int16))
        result["cpu_baseline"] = {
            "value": round(algo_bytes / med_s / 1e9, 2),
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"same workload (W=8 x 64 MiB bf16), torch CPU oracle, median of {nruns} passes, "
                      f"{med_s * 1e3:.1f} ms per pass",
            "host_cpus": os.cpu_count(),
            "gpu_matches_cpu_bitwise": bool(same),
        }
        # the same oracle on one thread (three passes), and what it ran on
        threads = torch.get_num_threads()
        torch.set_num_threads(1)
        one_s, _ = cpu_baseline(torch, bufs_cpu, 0.0)
        torch.set_num_threads(threads)
        model = ""
        try:
            with open("/proc/cpuinfo") as f:
                model = next((ln.split(":", 1)[1].strip() for ln in f if ln.startswith("model name")), "")
        except OSError:
            pass
        result["cpu_baseline"].update({
            "one_thread": {"value": round(algo_bytes / one_s / 1e9, 2), "unit": "GB/s",
                           "ms_per_pass": round(one_s * 1e3, 1)},
            "cpu_model": model, "torch_version": torch.__version__})
        del bufs_cpu

    if not args.no_other_ops:
        try:
            result["other_ops"] = other_ops(torch, tccl_amd, lib, device)
        except RuntimeError as e:        # the headline must still be printed
            result["other_ops"] = {"error": str(e)[:200]}

    if args.calibrate_copy:
        nbytes = 256 << 20
        src = torch.randint(-128, 128, (nbytes,), dtype=torch.int8, device=device)
        dst = torch.empty_like(src)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for _ in range(20):
            assert lib.tccl_tree_copy_step(src.data_ptr(), dst.data_ptr(), None, nbytes, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(src, dst)
        del src, dst

    if args.sweep:
        run_sweep(torch, tccl_amd, lib, device)

    print(json.dumps(result), flush=True)


def other_ops(torch, tccl_amd, lib, device):
    """The other operations of the path at their full benchmark shapes, bf16: GB/s on algorithmic
    bytes from HIP events (30 launches after 5 warm-ups).  Each rotates over enough disjoint
    buffers that nothing is served from the 256 MB memory-side cache."""
    import gc
    from tccl_amd import _lib
    out = {}
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    # reduce-scatter: W=8 inputs of 67,108,864 elements, every rank's share in turn (8 x 144 MiB touched)
    g = make_world(tccl_amd, torch, 8, 67_108_864, torch.bfloat16, device)
    turn = [0]

    def rs():
        turn[0] += 1
        return tccl_amd.reduce_scatter(g.tensor(turn[0] % 8))
    _, ms = time_steps(torch, lib, rs, 32, 8)
    out["reduce_scatter_w8_64Mi_el_gbs"] = round(9 * (67_108_864 // 8) * 2 / (ms * 1e-3) / 1e9, 1)
    tccl_amd.unregister(g)
    del g
    gc.collect()
    torch.cuda.empty_cache()

    # all-gather: W=8 x 8,388,608 elements, two groups alternating (2 x 256 MiB touched)
    gs = [make_world(tccl_amd, torch, 8, 8_388_608, torch.bfloat16, device) for _ in range(2)]

    def ag():
        turn[0] += 1
        return tccl_amd.all_gather(gs[turn[0] % 2].tensor(0), 8)
    _, ms = time_steps(torch, lib, ag, 30, 6)
    out["all_gather_w8_8Mi_el_gbs"] = round(2 * 8 * 8_388_608 * 2 / (ms * 1e-3) / 1e9, 1)
    for g in gs:
        tccl_amd.unregister(g)
    del gs
    gc.collect()
    torch.cuda.empty_cache()

    # tree node steps on 128 MiB halves in 128 KiB chunks: four different jobs in turn (2 GiB touched)
    half = 67_108_864
    bufs = [torch.randn(half, dtype=torch.float32, device=device).to(torch.bfloat16) for _ in range(12)]
    jobs = [(_lib.NodeJob * 1)() for _ in range(4)]

    def set_reduce():
        for i, j in enumerate(jobs):
            j[0].src[0], j[0].src[1], j[0].src[2] = bufs[3 * i + 1].data_ptr(), bufs[3 * i + 2].data_ptr(), bufs[3 * i].data_ptr()
            j[0].dst[0], j[0].dst[1] = bufs[3 * i].data_ptr(), None
            j[0].numel, j[0].is_copy = half, 0

    def set_copy():
        for i, j in enumerate(jobs):
            j[0].src[0], j[0].src[1], j[0].src[2] = bufs[3 * i].data_ptr(), None, None
            j[0].dst[0], j[0].dst[1] = bufs[3 * i + 1].data_ptr(), bufs[3 * i + 2].data_ptr()
            j[0].numel, j[0].is_copy = half, 1

    def level():
        turn[0] += 1
        return lib.tccl_tree_level(jobs[turn[0] % 4], 1, 0, 65_536, stream)
    set_reduce()
    _, ms = time_steps(torch, lib, level, 32, 8)
    out["tree_reduce_step_2_children_128MiB_gbs"] = round(4 * half * 2 / (ms * 1e-3) / 1e9, 1)
    set_copy()
    _, ms = time_steps(torch, lib, level, 32, 8)
    out["tree_copy_step_2_destinations_128MiB_gbs"] = round(3 * half * 2 / (ms * 1e-3) / 1e9, 1)
    del bufs
    gc.collect()
    torch.cuda.empty_cache()

    # whole double-tree all-reduce, W=8 x 256 MiB in 128 KiB chunks (4 GiB touched per call): the level
    # schedule (one launch per tree level) and the pipelined single launch (ranks signal each other per chunk)
    g = make_world(tccl_amd, torch, 8, 134_217_728, torch.bfloat16, device)
    _, ms = time_steps(torch, lib, lambda: tccl_amd.double_tree_all_reduce_world(g, fused=False, pipelined=False), 5, 2)
    out["double_tree_w8_256MiB_level_schedule_ms"] = round(ms, 3)
    _, ms = time_steps(torch, lib,
                       lambda: tccl_amd.double_tree_all_reduce_world(g, pipelined=True, chunk_elems=65_536), 5, 2)
    out["double_tree_w8_256MiB_pipelined_128KiB_chunks_ms"] = round(ms, 3)
    _, ms = time_steps(torch, lib, lambda: tccl_amd.double_tree_all_reduce_world(g, pipelined=True), 5, 2)
    out["double_tree_w8_256MiB_pipelined_32KiB_chunks_ms"] = round(ms, 3)
    out["double_tree_pipelined_expired_waits"] = tccl_amd.signal_pad_timeouts(g)
    tccl_amd.unregister(g)
    del g
    gc.collect()
    torch.cuda.empty_cache()

    # all W ranks' all-reduce in place in one launch (two-shot with the blockwise barrier), 8 x 64 MiB
    g = make_world(tccl_amd, torch, 8, 33_554_432, torch.bfloat16, device)
    _, ms = time_steps(torch, lib, lambda: tccl_amd.two_shot_all_reduce_world(g, with_outputs=False), 20, 5)
    out["two_shot_in_place_all_ranks_w8_64MiB_us"] = round(ms * 1e3, 1)
    out["two_shot_expired_waits"] = tccl_amd.signal_pad_timeouts(g)
    tccl_amd.unregister(g)
    del g
    gc.collect()
    torch.cuda.empty_cache()
    return out


def run_sweep(torch, tccl_amd, lib, device):
    """Every op at its full benchmark shape and the all-reduce size sweep; JSON lines on
    stderr (GB/s on algorithmic bytes from HIP events; p50 us per launch)."""
    import gc

    def emit(**kw):
        print(json.dumps(kw), file=sys.stderr, flush=True)

    def rate(fn, nbytes, steps=50, warmup=10):
        _, dev_ms = time_steps(torch, lib, fn, steps, warmup)
        return round(nbytes / (dev_ms * 1e-3) / 1e9, 1), round(dev_ms * 1e3, 2)

    def drop(g):
        tccl_amd.unregister(g)
        gc.collect()
        torch.cuda.empty_cache()

    # all-reduce sweep: W in {2,4,8}, 16 KiB .. 256 MiB per buffer in powers of 4
    for world in (2, 4, 8):
        g = make_world(tccl_amd, torch, world, (256 << 20) // 2, torch.bfloat16, device)
        nbytes = 16 << 10
        while nbytes <= (256 << 20):
            view = g.tensor(0)[:nbytes // 2]
            fn = lambda: tccl_amd.one_shot_all_reduce(view)
            gbs, us = rate(fn, (world + 1) * nbytes)
            p50, _ = latency_p50_us(torch, lib, fn, reps=200, warmup=10)
            emit(op="all_reduce", world=world, dtype="bf16", bytes_per_buffer=nbytes, gbs=gbs, avg_us=us,
                 p50_us=round(p50, 2))
            nbytes *= 4
        drop(g)

    # reduce-scatter, rank 3 of 8, 67,108,864 elements per input
    for dtype, name in ((torch.bfloat16, "bf16"), (torch.float32, "f32")):
        g = make_world(tccl_amd, torch, 8, 67_108_864, dtype, device)
        t = g.tensor(3)
        per_bytes = t.numel() // 8 * t.element_size()
        gbs, us = rate(lambda: tccl_amd.reduce_scatter(t), 9 * per_bytes)
        emit(op="reduce_scatter", world=8, rank=3, dtype=name, numel=t.numel(), gbs=gbs, avg_us=us)
        drop(g)

    # all-gather pack, 8 x 8,388,608 elements
    for dtype, name in ((torch.bfloat16, "bf16"), (torch.float32, "f32"), (torch.int8, "int8")):
        g = make_world(tccl_amd, torch, 8, 8_388_608, dtype, device)
        t = g.tensor(0)
        gbs, us = rate(lambda: tccl_amd.all_gather(t, 8), 2 * 8 * t.numel() * t.element_size())
        emit(op="all_gather", world=8, dtype=name, numel=t.numel(), gbs=gbs, avg_us=us)
        drop(g)

    # double-tree node step on one 128 MiB half in 128 KiB chunks: reduce (own + 2 children,
    # in place) and forward copy (parent -> own + output), via the level launcher
    from tccl_amd import _lib
    half = 67_108_864
    bufs = [torch.randn(half, dtype=torch.float32, device=device).to(torch.bfloat16) for _ in range(5)]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    job = (_lib.NodeJob * 1)()
    for c in (0, 1, 2):
        kids = [bufs[1].data_ptr() if c >= 1 else None, bufs[2].data_ptr() if c >= 2 else None]
        job[0].src[0], job[0].src[1], job[0].src[2] = kids[0], kids[1], bufs[0].data_ptr()
        job[0].dst[0], job[0].dst[1] = bufs[0].data_ptr(), None
        job[0].numel, job[0].is_copy = half, 0
        gbs, us = rate(lambda: lib.tccl_tree_level(job, 1, 0, 65_536, stream), (c + 2) * half * 2)
        emit(op="tree_reduce_step", children=c, chunk_bytes=131072, bytes_per_half=half * 2, gbs=gbs, avg_us=us)
    for ndst in (1, 2):
        job[0].src[0], job[0].src[1], job[0].src[2] = bufs[0].data_ptr(), None, None
        job[0].dst[0], job[0].dst[1] = bufs[3].data_ptr(), bufs[4].data_ptr() if ndst == 2 else None
        job[0].numel, job[0].is_copy = half, 1
        gbs, us = rate(lambda: lib.tccl_tree_level(job, 1, 0, 65_536, stream), (1 + ndst) * half * 2)
        emit(op="tree_copy_step", destinations=ndst, chunk_bytes=131072, bytes_per_half=half * 2, gbs=gbs, avg_us=us)
    del bufs
    gc.collect()
    torch.cuda.empty_cache()

    # whole double-tree all-reduce, W=8 x 256 MiB
    g = make_world(tccl_amd, torch, 8, 134_217_728, torch.bfloat16, device)
    _, dev_ms = time_steps(torch, lib, lambda: tccl_amd.double_tree_all_reduce_world(g, fused=False, pipelined=False), 5, 2)
    emit(op="double_tree_all_reduce", world=8, bytes_per_buffer=256 << 20, schedule="one launch per tree level",
         ms=round(dev_ms, 3))
    for chunk_kib in (128, 32):
        _, dev_ms = time_steps(torch, lib, lambda: tccl_amd.double_tree_all_reduce_world(
            g, pipelined=True, chunk_elems=chunk_kib * 512), 5, 2)
        emit(op="double_tree_all_reduce", world=8, bytes_per_buffer=256 << 20,
             schedule=f"one persistent launch, ranks signal each other per {chunk_kib} KiB chunk",
             ms=round(dev_ms, 3), expired_waits=tccl_amd.signal_pad_timeouts(g))
    drop(g)

    # every rank's all-reduce in one launch (two-shot with the blockwise barrier), W=8 x 64 MiB
    g = make_world(tccl_amd, torch, 8, 33_554_432, torch.bfloat16, device)
    for with_outputs in (False, True):
        _, dev_ms = time_steps(torch, lib,
                               lambda: tccl_amd.two_shot_all_reduce_world(g, with_outputs=with_outputs), 20, 5)
        nbytes = ((3 if not with_outputs else 4) * 8 - 1) * 33_554_432 * 2
        emit(op="two_shot_all_reduce_all_ranks", world=8, bytes_per_buffer=64 << 20, outputs=with_outputs,
             avg_us=round(dev_ms * 1e3, 1), gbs=round(nbytes / (dev_ms * 1e-3) / 1e9, 1),
             expired_waits=tccl_amd.signal_pad_timeouts(g))
    drop(g)


if __name__ == "__main__":
    main()
