#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the one the headline metric is quoted on): one-shot all-reduce (sum) over W=8
virtual-rank buffers of 64 MiB bf16 each (33,554,432 elements, buffer r made on the CPU by
``torch.manual_seed(r); torch.randn(n, dtype=bfloat16)``), all resident in HBM before the
timed region.  A step is one call of ``tccl_amd.one_shot_all_reduce`` (output allocation from
torch's caching allocator plus one kernel launch through the C ABI).  Prints ONE JSON line on
stdout.

Algorithmic bytes per step: (W + 1) * N * 2 = 603,979,776 (W*N read, N written).

Besides the headline the line carries: the same step rotated over 8 buffer sets (nothing
served from the 256 MB memory-side cache), the memory system's own read-pass and write-pass
times, latencies at 1 MiB (single launch, launch floor, graph replay), the torch CPU oracle
timed on the host, every other operation of the path at its benchmark shape (cold), and a
compact size sweep.  ``--only OP`` runs one operation alone, for profiler runs whose kernel
statistics must hold one kernel at one size.
"""
from __future__ import annotations

import argparse
import ctypes
import gc
import hashlib
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
COLD_BYTES = 1 << 30            # a rotation touches at least this much between two uses of a byte (cache: 256 MB)
MIN_SETS = 4                    # ... over at least this many disjoint buffer sets
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "headline_traffic.json")
# What a launch of 512 x 256 lanes lasts that loads and stores ONE vector per lane from cold memory (rocprofv3,
# profiles/probe_kernels_fixed_cost_of_a_short_cold_launch.txt; `bench.py --only floor` measures it again):
# the part of a short kernel's time that does not depend on its bytes.
LAUNCH_COST_US = 2.6

ONLY_OPS = ["all_reduce", "all_reduce_rotated", "probe_read", "probe_write", "reduce_scatter_bf16", "reduce_scatter_f32",
            "all_gather_bf16", "all_gather_f32", "all_gather_int8", "tree_reduce_c0", "tree_reduce_c1",
            "tree_reduce_c2", "tree_copy_1", "tree_copy_2", "double_tree_level", "double_tree_pipelined",
            "double_tree_pipelined_drawn", "two_shot", "two_shot_drawn", "copy_calibration", "placement", "ceilings", "phase_timing", "floor"]
# the all-reduce at the sizes of the sweep, rotated cold as the sweep does: c1 = the CPU-runnable shape (W=8 x 8 MiB)
SWEEP_OPS = {"c1": (8, 8)}
SWEEP_OPS.update({f"all_reduce_w{w}_{m}MiB": (w, m) for w in (2, 4, 8) for m in (4, 16, 64, 256)})
ONLY_OPS += list(SWEEP_OPS)


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20, help="untimed steps right before the timed ones")
    p.add_argument("--preheat", type=int, default=300,
                   help="launches of the headline step before the warm-up, reported as preheat_launches: "
                        "the first 100 or so launches after an idle period run 1-2 %% slower while the clocks settle, "
                        "so a short --warmup would time the ramp")
    p.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timing")
    p.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU work budget for the baseline leg")
    p.add_argument("--no-other-ops", action="store_true",
                   help="skip reduce-scatter, all-gather, the tree node steps and the signalling kernels")
    p.add_argument("--no-sweep", action="store_true", help="skip the size sweep")
    p.add_argument("--no-ipc", action="store_true", help="skip the leg with one process per rank")
    p.add_argument("--calibrate-copy", action="store_true",
                   help="also run 20 plain copies of 256 MiB (tccl_tree_copy_step), so that a rocprofv3 --pmc "
                        "run of this command holds a kernel of known traffic to scale the counters by")
    p.add_argument("--only", choices=ONLY_OPS,
                   help="run this one operation alone (--steps launches after --warmup) and print a small JSON line")
    p.add_argument("--stamps", action="store_true",
                   help="with --only OP: run OP through benchlib/libtccl_amd_stamped.so (the library's own kernels with "
                        "wall-clock stamps per workgroup) and print when the workgroups start, get their first data, finish "
                        "reading and finish writing, per XCD")
    return p.parse_args()


# ------------------------------------------------------------------------------------------ timing helpers

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


def raw_stream(torch):
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def time_steps(torch, lib, fn, steps, warmup):
    """(wall ms per step, HIP-event ms per step) over exactly `steps` calls."""
    stream = raw_stream(torch)
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
    """Median (and 99th percentile) over single-launch HIP-event pairs."""
    stream = raw_stream(torch)
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


def free(torch):
    gc.collect()
    torch.cuda.empty_cache()


class Rotation:
    """Calls fn(k) for k = 0, 1, ..., nsets-1, 0, ...: one launch per call, each on its own set of
    buffers, so that `nsets` x bytes_per_set (>= COLD_BYTES) lie between two uses of a byte."""

    def __init__(self, fn, nsets):
        self.fn, self.nsets, self.turn = fn, nsets, 0

    def __call__(self):
        self.turn += 1
        return self.fn(self.turn % self.nsets)


def sets_for(bytes_per_set):
    return max(MIN_SETS, -(-COLD_BYTES // bytes_per_set))


# ------------------------------------------------------------------------------------------ inputs

def cpu_recipe(torch, world, numel, dtype):
    """The baseline's input recipe: buffer r = manual_seed(r); randn(n, dtype) made on the CPU."""
    out = []
    for r in range(world):
        torch.manual_seed(r)
        out.append(torch.randn(numel, dtype=dtype))
    return out


class Noise:
    """One block of device-made N(0,1) values (seeded) from which timing-only buffers are filled:
    values do not matter to a streaming kernel's time, and making 20 GB of them would."""

    def __init__(self, torch, device, nbytes=256 << 20):
        gen = torch.Generator(device=device)
        gen.manual_seed(1234)
        self.torch = torch
        self.f32 = torch.randn(nbytes // 4, dtype=torch.float32, device=device, generator=gen)
        self.bf16 = self.f32[: nbytes // 8].to(torch.bfloat16)     # nbytes/4 bytes of bf16

    def fill(self, t, salt=0):
        """t <- noise of t's dtype (int8: the raw bytes), starting at a salt-dependent offset."""
        torch = self.torch
        if t.dtype == torch.bfloat16:
            src = self.bf16
        elif t.dtype == torch.float32:
            src = self.f32
        else:
            src = self.f32.view(torch.int8)
        n, m = t.numel(), src.numel()
        flat = t.view(-1)
        off = (salt * 4099 * 8) % max(1, m // 2)
        done = 0
        while done < n:
            take = min(n - done, m - off)
            flat[done:done + take].copy_(src[off:off + take])
            done += take
            off = 0
        return t


def make_world(tccl_amd, torch, noise, world, numel, dtype, device, salt=0):
    group = tccl_amd.empty_world(world, numel, dtype, device)
    for r in range(world):
        noise.fill(group.tensor(r), salt + r)
    return group


# ------------------------------------------------------------------------------------------ CPU baseline

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


# ------------------------------------------------------------------------------------------ single operations

class Ops:
    """Every operation of the path at its benchmark shape, each as (callable doing ONE launch on
    rotated buffers, algorithmic bytes per launch, kernel it launches)."""

    def __init__(self, torch, tccl_amd, lib, plib, noise, device):
        self.torch, self.tccl_amd, self.lib, self.plib, self.noise, self.device = torch, tccl_amd, lib, plib, noise, device
        self.keep = []

    def close(self):
        for g in self.keep:
            if hasattr(g, "world_size"):
                self.tccl_amd.unregister(g)
        self.keep = []
        free(self.torch)

    def _worlds(self, nsets, world, numel, dtype):
        gs = [make_world(self.tccl_amd, self.torch, self.noise, world, numel, dtype, self.device, salt=17 * k)
              for k in range(nsets)]
        self.keep += gs
        return gs

    def all_reduce(self, rotated):
        torch, numel = self.torch, BYTES_PER_BUF // 2
        nbytes = (WORLD + 1) * BYTES_PER_BUF
        nsets = sets_for(nbytes) if rotated else 1
        nsets = max(nsets, 8) if rotated else 1
        gs = self._worlds(nsets, WORLD, numel, torch.bfloat16)
        outs = [torch.empty_like(g.tensor(0)) for g in gs]
        fn = Rotation(lambda k: self.tccl_amd.one_shot_all_reduce(gs[k].tensor(0), out=outs[k]), nsets)
        return fn, nbytes, "sum_phased_skewed_kernel<Bf16Sum, 8>"

    def all_reduce_cold(self, world, mib):
        """The sweep's protocol: W buffers of `mib` MiB bf16 through the C entry point, rotated over
        enough buffer sets that COLD_BYTES lie between two uses of a byte."""
        torch, nbytes = self.torch, mib << 20
        numel = nbytes // 2
        touched = (world + 1) * nbytes
        nsets = sets_for(touched)
        sets = []
        for k in range(nsets):
            bufs = [self.noise.fill(torch.empty(numel, dtype=torch.bfloat16, device=self.device), 13 * k + r)
                    for r in range(world)]
            o = torch.empty(numel, dtype=torch.bfloat16, device=self.device)
            sets.append((bufs, o, ctypes.cast((ctypes.c_void_p * world)(*[b.data_ptr() for b in bufs]),
                                               ctypes.POINTER(ctypes.c_void_p))))
        self.keep.append(sets)
        stream = raw_stream(torch)
        fn = Rotation(lambda k: self.lib.tccl_all_reduce_sum(sets[k][2], world, sets[k][1].data_ptr(), numel, 0, stream), nsets)
        return fn, touched, "sum_phased*_kernel<Bf16Sum, %d, ...>" % world

    def probe_read(self):
        torch = self.torch
        gs = self._worlds(1, WORLD, BYTES_PER_BUF // 2, torch.bfloat16)
        sink = torch.zeros(4096, dtype=torch.uint8, device=self.device)
        s = raw_stream(torch)
        fn = lambda: self.plib.tccl_probe_read(gs[0].ptr_array, WORLD, BYTES_PER_BUF, sink.data_ptr(), s)
        self.keep.append(sink)
        return fn, WORLD * BYTES_PER_BUF, "probe_read_kernel<8>"

    def probe_write(self):
        torch = self.torch
        out = torch.empty(BYTES_PER_BUF, dtype=torch.uint8, device=self.device)
        s = raw_stream(torch)
        self.keep.append(out)
        return (lambda: self.plib.tccl_probe_write(out.data_ptr(), BYTES_PER_BUF, s)), BYTES_PER_BUF, "probe_write_kernel"

    def reduce_scatter(self, dtype):
        """W=8 inputs of 67,108,864 elements, rank 3's share (the baseline's shape); two input sets
        alternate and the share is written to rotating outputs: 2 x 8 x 16 MiB of input shares
        (bf16) cannot be held by the cache together with everything else that is touched."""
        torch, numel = self.torch, 67_108_864
        esize = 2 if dtype == torch.bfloat16 else 4
        per = numel // WORLD
        nbytes = (WORLD + 1) * per * esize
        nsets = sets_for(nbytes)
        gs = self._worlds(nsets, WORLD, numel, dtype)
        outs = [torch.empty(per, dtype=dtype, device=self.device) for _ in range(nsets)]
        fn = Rotation(lambda k: self.tccl_amd.reduce_scatter(gs[k].tensor(3), out=outs[k]), nsets)
        return fn, nbytes, "sum_phased_kernel<%s, 8, ...>" % ("Bf16Sum" if esize == 2 else "F32Sum")

    def all_gather(self, dtype):
        torch, numel = self.torch, 8_388_608
        esize = torch.empty(0, dtype=dtype).element_size()
        nbytes = 2 * WORLD * numel * esize
        nsets = sets_for(nbytes)
        gs = self._worlds(nsets, WORLD, numel, dtype)
        outs = [torch.empty((WORLD, numel), dtype=dtype, device=self.device) for _ in range(nsets)]
        fn = Rotation(lambda k: self.tccl_amd.all_gather(gs[k].tensor(0), WORLD, out=outs[k]), nsets)
        return fn, nbytes, "pack_kernel"

    def tree_step(self, children=None, destinations=None):
        """One node step on a 128 MiB half in 128 KiB chunks through the level launcher: a reduce
        step (own + `children` child buffers, in place) or a copy step (parent -> `destinations`)."""
        from tccl_amd import _lib
        torch, half = self.torch, 67_108_864
        nbuf = (children + 1) if children is not None else (destinations + 1)
        nbytes = ((children + 2) if children is not None else (1 + destinations)) * half * 2
        nsets = sets_for(nbuf * half * 2)
        jobs = []
        for k in range(nsets):
            bufs = [self.noise.fill(torch.empty(half, dtype=torch.bfloat16, device=self.device), 31 * k + i)
                    for i in range(nbuf)]
            self.keep += bufs
            j = (_lib.NodeJob * 1)()
            if children is not None:
                kids = [bufs[1].data_ptr() if children >= 1 else None, bufs[2].data_ptr() if children >= 2 else None]
                j[0].src[0], j[0].src[1], j[0].src[2] = kids[0], kids[1], bufs[0].data_ptr()
                j[0].dst[0], j[0].dst[1] = bufs[0].data_ptr(), None
                j[0].numel, j[0].is_copy = half, 0
            else:
                j[0].src[0], j[0].src[1], j[0].src[2] = bufs[0].data_ptr(), None, None
                j[0].dst[0], j[0].dst[1] = bufs[1].data_ptr(), bufs[2].data_ptr() if destinations == 2 else None
                j[0].numel, j[0].is_copy = half, 1
            jobs.append(j)
        s = raw_stream(torch)
        fn = Rotation(lambda k: self.lib.tccl_tree_level(jobs[k], 1, 0, 65_536, s), nsets)
        return fn, nbytes, "tree_level_kernel / tree_copy_level_kernel"

    def double_tree(self, how):
        """Whole double-tree all-reduce, W=8 x 256 MiB (4 GiB touched per call)."""
        torch = self.torch
        gs = self._worlds(1, WORLD, 134_217_728, torch.bfloat16)
        g = gs[0]
        t = self.tccl_amd
        if how == "level":
            fn = lambda: t.double_tree_all_reduce_world(g, fused=False, pipelined=False)
        elif how == "pipelined_128k":
            fn = lambda: t.double_tree_all_reduce_world(g, pipelined=True, chunk_elems=65_536)
        else:
            fn = lambda: t.double_tree_all_reduce_world(g, pipelined=True, draw_places=(how == "pipelined_drawn"))
        return fn, 74 * (128 << 20), "tree_level_kernel x 6 / tree_pipelined_kernel", g

    def two_shot(self, drawn=False):
        torch = self.torch
        gs = self._worlds(1, WORLD, BYTES_PER_BUF // 2, torch.bfloat16)
        g = gs[0]
        fn = lambda: self.tccl_amd.two_shot_all_reduce_world(g, with_outputs=False, draw_places=drawn)
        return fn, (3 * WORLD - 1) * BYTES_PER_BUF, "two_shot_kernel<Bf16Sum, 8>", g

    def copy_calibration(self):
        torch, nbytes = self.torch, 256 << 20
        src = torch.randint(-128, 128, (nbytes,), dtype=torch.int8, device=self.device)
        dst = torch.empty_like(src)
        s = raw_stream(torch)
        self.keep += [src, dst]
        return (lambda: self.lib.tccl_tree_copy_step(src.data_ptr(), dst.data_ptr(), None, nbytes, s)), 2 * nbytes, "copy_kernel"

    def get(self, name):
        torch = self.torch
        if name in SWEEP_OPS:
            return self.all_reduce_cold(*SWEEP_OPS[name])
        if name == "all_reduce":
            return self.all_reduce(False)
        if name == "all_reduce_rotated":
            return self.all_reduce(True)
        if name in ("probe_read", "probe_write", "copy_calibration"):
            return getattr(self, name)()
        if name.startswith("reduce_scatter_"):
            return self.reduce_scatter(torch.bfloat16 if name.endswith("bf16") else torch.float32)
        if name.startswith("all_gather_"):
            return self.all_gather({"bf16": torch.bfloat16, "f32": torch.float32, "int8": torch.int8}[name[11:]])
        if name.startswith("tree_reduce_c"):
            return self.tree_step(children=int(name[-1]))
        if name.startswith("tree_copy_"):
            return self.tree_step(destinations=int(name[-1]))
        if name == "double_tree_level":
            return self.double_tree("level")[:3]
        if name == "double_tree_pipelined":
            return self.double_tree("pipelined")[:3]
        if name == "double_tree_pipelined_drawn":
            return self.double_tree("pipelined_drawn")[:3]
        if name in ("two_shot", "two_shot_drawn"):
            return self.two_shot(name.endswith("drawn"))[:3]
        raise ValueError(name)


def cold_ceilings(torch, lib, plib, device):
    """What the memory system gives the simplest kernels on data that is in no cache (4 GiB arena,
    every launch on the next 512 MiB of it): the reference points for the operations' own rates."""
    arena = torch.empty(4 << 30, dtype=torch.uint8, device=device)
    arena.view(torch.int32).fill_(0x3C003C00)
    sink = torch.zeros(4096, dtype=torch.uint8, device=device)
    s = raw_stream(torch)
    base = arena.data_ptr()
    R = 512 << 20
    out = {}
    _, ms = time_steps(torch, lib, Rotation(lambda k: plib.tccl_probe_read_dense(base + k * R, R, sink.data_ptr(), s), 8), 32, 16)
    out["read_dense_gbs"] = round(R / (ms * 1e-3) / 1e9, 1)
    ptrs = [(ctypes.c_void_p * 8)(*[base + k * R + i * (64 << 20) for i in range(8)]) for k in range(8)]
    _, ms = time_steps(torch, lib, Rotation(lambda k: plib.tccl_probe_read(ptrs[k], 8, 64 << 20, sink.data_ptr(), s), 8), 32, 16)
    out["read_8_streams_128KiB_tiles_gbs"] = round(R / (ms * 1e-3) / 1e9, 1)
    W = 64 << 20
    _, ms = time_steps(torch, lib, Rotation(lambda k: plib.tccl_probe_write(base + k * W, W, s), 64), 128, 64)
    out["write_64MiB_128KiB_tiles_gbs"] = round(W / (ms * 1e-3) / 1e9, 1)
    _, ms = time_steps(torch, lib, Rotation(lambda k: plib.tccl_probe_write_small(base + k * W, W, s), 64), 128, 64)
    out["write_64MiB_32KiB_tiles_gbs"] = round(W / (ms * 1e-3) / 1e9, 1)
    D = 256 << 20
    _, ms = time_steps(torch, lib, Rotation(lambda k: plib.tccl_probe_write_dense(base + k * D, D, s), 16), 48, 16)
    out["write_256MiB_one_dense_window_gbs"] = round(D / (ms * 1e-3) / 1e9, 1)
    C = 128 << 20
    _, ms = time_steps(torch, lib, Rotation(lambda k: plib.tccl_probe_copy(base + (2 * k) * C, base + (2 * k + 1) * C, C, s), 16), 32, 16)
    out["copy_128MiB_gbs"] = round(2 * C / (ms * 1e-3) / 1e9, 1)
    out["note"] = "benchlib/probe.hip kernels on a 4 GiB arena, every launch on the next part of it (nothing cached)"
    del arena
    free(torch)
    return out


def phase_timing(torch, tccl_amd, plib, device, launches=48):
    """When do the workgroups of the large all-reduce finish reading and writing?  The kernel's
    shape with wall-clock stamps per workgroup, rotated over 8 buffer sets; printed per XCD and
    for the first and the second workgroup that a compute unit receives (workgroups b and b + 256)."""
    noise = Noise(torch, device)
    numel = BYTES_PER_BUF // 2
    gs = [make_world(tccl_amd, torch, noise, WORLD, numel, torch.bfloat16, device, salt=9 * k) for k in range(8)]
    outs = [torch.empty(numel, dtype=torch.bfloat16, device=device) for _ in range(8)]
    ntiles = BYTES_PER_BUF // (128 << 10)
    stamps = torch.zeros((launches, ntiles, 3), dtype=torch.int64, device=device)
    s = raw_stream(torch)
    for i in range(launches):
        assert plib.tccl_probe_sum_timed(gs[i % 8].ptr_array, outs[i % 8].data_ptr(), BYTES_PER_BUF, stamps[i].data_ptr(), s) == 0
    torch.cuda.synchronize()
    t = stamps[16:].cpu().double()                            # skip the first 16 launches
    t = (t - t[:, :, 0].min(dim=1, keepdim=True)[0].unsqueeze(-1)) * 0.01       # us after the launch's first start
    b = torch.arange(ntiles)
    print(f"W=8 x 64 MiB bf16, {ntiles} tiles of 128 KiB, mean over {t.shape[0]} launches rotated over 8 buffer sets; "
          f"span {float(t[:, :, 2].max(dim=1)[0].mean()):.2f} us; times in us after the launch's first workgroup started")
    print("XCD  workgroup on its unit   read-end mean   read-end max   write-end mean   write-end max")
    for x in range(8):
        for second in (0, 1):
            sel = (b % 8 == x) & ((b >= ntiles // 2) == bool(second))
            rd, wr = t[:, sel, 1], t[:, sel, 2]
            print(f"{x:3d}  {'second' if second else 'first ':6s}              {float(rd.mean()):10.2f}   {float(rd.max(dim=1)[0].mean()):12.2f}   "
                  f"{float(wr.mean()):13.2f}   {float(wr.max(dim=1)[0].mean()):12.2f}")
    for g in gs:
        tccl_amd.unregister(g)


class _DeviceWords:
    """Device memory that torch does not own, seen through ``__cuda_array_interface__``."""

    def __init__(self, ptr, nbytes):
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (ptr, False), "version": 2}


def stamp_table(args, torch, tccl_amd, lib, device, burst=8):
    """--only OP --stamps: OP through the stamped build of the library (every kernel of the library records
    the 100 MHz wall clock per workgroup: start, first iteration's data there, last load reduced, last store
    acknowledged).  Launches go out in bursts of `burst` back to back (rotating over the operation's buffer
    sets as always); the stamps of a burst's last launch are read after it, `--steps` bursts in all."""
    ptr, slots, room = ctypes.c_void_p(), ctypes.c_int(), ctypes.c_int()
    assert lib.tccl_stamp_buffer(ctypes.byref(ptr), ctypes.byref(slots), ctypes.byref(room)) == 0
    words = torch.as_tensor(_DeviceWords(ptr.value, 8 * slots.value * room.value), device=device).view(torch.int64)
    words = words.view(room.value, slots.value)
    noise = Noise(torch, device)
    ops = Ops(torch, tccl_amd, lib, None, noise, device)
    fn, nbytes, kernel = ops.get(args.only)
    stream = raw_stream(torch)
    ev = HipEvents(lib, 2)
    for _ in range(max(args.warmup, burst)):
        fn()
    tables, event_us = [], []
    for _ in range(args.steps):
        words.zero_()
        torch.cuda.synchronize()
        ev.record(0, stream)
        for _ in range(burst):
            fn()
        ev.record(1, stream)
        torch.cuda.synchronize()
        event_us.append(ev.elapsed_ms(0, 1) * 1e3 / burst)
        w = words.cpu()
        tables.append(w[w[:, 0] != 0].double())
    ev.close()
    n = min(t.shape[0] for t in tables)
    assert all(t.shape[0] == n for t in tables), "the operation's launches differ in their grids"
    t = torch.stack(tables)                                              # [bursts, workgroups, 4]
    t = (t - t[:, :, 0].min(dim=1, keepdim=True)[0].unsqueeze(-1)) * 0.01      # us after the launch's first start
    for slot in (1, 2):                                                  # kernels without those marks leave zeros
        if float(tables[0][:, slot].max()) == 0.0:
            t[:, :, slot] = float("nan")
    span = t[:, :, 3].max(dim=1)[0]
    b = torch.arange(n)
    cus = 256
    rounds = max(1, -(-n // cus))
    print(f"Operation: bench.py --only {args.only} --stamps --steps {args.steps} --warmup {args.warmup}   kernel: {kernel}")
    print(f"{n} workgroups stamped in the last launch of each burst of {burst} back-to-back calls, mean over {args.steps} bursts; "
          f"algorithmic bytes per call {nbytes:,}")
    print(f"HIP events over a burst: {statistics.mean(event_us):.2f} us per call (min {min(event_us):.2f}, max {max(event_us):.2f})")
    print(f"first workgroup's start to last store acknowledged: mean {float(span.mean()):.2f} us, min {float(span.min()):.2f}, "
          f"max {float(span.max()):.2f}   -> {nbytes / float(span.mean()) / 1e3:.0f} GB/s inside the launch")
    if rounds > 1 and float(t[:, b // cus == 1, 0].mean()) > 0.2 * float(span.mean()):
        print("NOTE: the second workgroup of a compute unit started only when the first had finished: the stamped build of this kernel "
              "needs more registers than the product's and does not fit two per unit, so this table does not show the product's launch")
    print("times in us after the launch's first workgroup started; 'k-th on its unit' = workgroup index // 256")
    print("XCD  k-th on its unit   start mean  start max | first data mean   max | last load reduced mean    max | last store acked mean    max")
    for x in range(8):
        for k in range(rounds):
            sel = (b % 8 == x) & (b // cus == k)
            if int(sel.sum()) == 0:
                continue
            c = [t[:, sel, i] for i in range(4)]
            f = lambda v: float(v.mean())
            m = lambda v: float(v.max(dim=1)[0].mean())
            print(f"{x:3d}  {k:3d}              {f(c[0]):10.2f}  {m(c[0]):9.2f} | {f(c[1]):15.2f} {m(c[1]):7.2f} | "
                  f"{f(c[2]):22.2f} {m(c[2]):7.2f} | {f(c[3]):21.2f} {m(c[3]):7.2f}")
    allf = lambda i: float(t[:, :, i].mean())
    allm = lambda i: float(t[:, :, i].max(dim=1)[0].mean())
    print(f"all                   {allf(0):10.2f}  {allm(0):9.2f} | {allf(1):15.2f} {allm(1):7.2f} | "
          f"{allf(2):22.2f} {allm(2):7.2f} | {allf(3):21.2f} {allm(3):7.2f}")
    ops.close()


def floor(args, torch, lib, plib, device):
    """What a short streaming kernel costs whatever it moves: an empty grid of 512 x 256 lanes, and the
    same grid with every lane loading one vector and storing it (data that is in no cache)."""
    arena = torch.empty(2 << 30, dtype=torch.uint8, device=device)
    arena.view(torch.int32).fill_(0x3C003C00)
    s = raw_stream(torch)
    base, half, step = arena.data_ptr(), 1 << 30, 4 << 20
    line = {"only": "floor", "steps": args.steps, "warmup": args.warmup}
    for wgs in (256, 512):
        _, ms = time_steps(torch, lib, lambda: plib.tccl_probe_empty_grid(wgs, s), args.steps, args.warmup)
        line[f"empty_grid_{wgs}_us"] = round(ms * 1e3, 2)
        fn = Rotation(lambda k: plib.tccl_probe_touch(base + k * step, base + half + k * step, wgs, s), half // step)
        _, ms = time_steps(torch, lib, fn, args.steps, args.warmup)
        line[f"touch_{wgs}_us"] = round(ms * 1e3, 2)
    print(json.dumps(line), flush=True)


def run_only(args, torch, tccl_amd, lib, plib, device):
    if args.only == "floor":
        return floor(args, torch, lib, plib, device)
    if args.stamps:
        return stamp_table(args, torch, tccl_amd, lib, device)
    if args.only == "placement":
        return placement(torch, plib, device)
    if args.only == "phase_timing":
        return phase_timing(torch, tccl_amd, plib, device)
    if args.only == "ceilings":
        print(json.dumps({"only": "ceilings", **cold_ceilings(torch, lib, plib, device)}), flush=True)
        return
    noise = Noise(torch, device)
    ops = Ops(torch, tccl_amd, lib, plib, noise, device)
    fn, nbytes, kernel = ops.get(args.only)
    _, ms = time_steps(torch, lib, fn, args.steps, args.warmup)
    line = {"only": args.only, "kernel": kernel, "steps": args.steps, "warmup": args.warmup,
            "avg_launch_us": round(ms * 1e3, 2), "algorithmic_bytes": nbytes,
            "gbs": round(nbytes / (ms * 1e-3) / 1e9, 1), "frac_of_8TBs": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    ops.close()
    if args.calibrate_copy:
        calibrate_copy(torch, lib, device)
    print(json.dumps(line), flush=True)


def calibrate_copy(torch, lib, device):
    nbytes = 256 << 20
    src = torch.randint(-128, 128, (nbytes,), dtype=torch.int8, device=device)
    dst = torch.empty_like(src)
    stream = raw_stream(torch)
    for _ in range(20):
        assert lib.tccl_tree_copy_step(src.data_ptr(), dst.data_ptr(), None, nbytes, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(src, dst)


def placement(torch, plib, device):
    """Where the hardware puts the workgroups of grids of 4 and 6 per compute unit."""
    for n in (1024, 1536):
        where = torch.full((2 * n,), -1, dtype=torch.int32, device=device)
        assert plib.tccl_probe_placement(where.data_ptr(), n, 20000, raw_stream(torch)) == 0
        torch.cuda.synchronize()
        w = where.cpu().view(n, 2)
        hw, xcc = w[:, 0], w[:, 1] & 15
        b = torch.arange(n)
        print(f"grid {n}: workgroups on XCD (index mod 8): {int((xcc == b % 8).sum())} of {n}")
        cu = (xcc << 16) | (hw & 0xFF00)
        per = torch.unique(cu, return_counts=True)[1]
        print(f"grid {n}: distinct compute units {per.numel()}, workgroups per unit min {int(per.min())} max {int(per.max())}")
        if n == 1024:
            for x in (0, 1):
                seq = [int(v) for v in hw[x::8][:64]]
                print(f"XCD {x}, i-th workgroup -> se.cu:", " ".join(f"{(v >> 13) & 7}.{(v >> 8) & 15}" for v in seq))


# ------------------------------------------------------------------------------------------ sweep

def sweep(torch, tccl_amd, lib, noise, device):
    """The all-reduce size sweep of the baseline (W in {2,4,8}, 16 KiB .. 256 MiB per buffer in
    powers of 4) through the C entry point on separate allocations: p50 us of single launches
    up to 1 MiB, GB/s on algorithmic bytes from 4 MiB, rotated over enough buffer sets (at least
    MIN_SETS) that COLD_BYTES lie between two uses of a byte.  Also the CPU-runnable shape (W=8 x 8 MiB), cold."""
    out = {"note": "all-reduce, bf16, C entry point; p50_us: single launches on one buffer set; "
                   "cold_gbs: algorithmic bytes / mean launch time, rotated over `sets` buffer sets (>= 4 sets and >= 1 GiB "
                   "touched between two uses of a byte)"}
    stream = raw_stream(torch)
    sizes = [16 << 10 << (2 * i) for i in range(8)]

    def one(world, nbytes, steps):
        numel = nbytes // 2
        touched = (world + 1) * nbytes
        nsets = 1 if nbytes <= (1 << 20) else sets_for(touched)
        sets = []
        for k in range(nsets):
            bufs = [noise.fill(torch.empty(numel, dtype=torch.bfloat16, device=device), 13 * k + r) for r in range(world)]
            o = torch.empty(numel, dtype=torch.bfloat16, device=device)
            sets.append((bufs, o, ctypes.cast((ctypes.c_void_p * world)(*[b.data_ptr() for b in bufs]),
                                               ctypes.POINTER(ctypes.c_void_p))))
        fn = Rotation(lambda k: lib.tccl_all_reduce_sum(sets[k][2], world, sets[k][1].data_ptr(), numel, 0, stream), nsets)
        if nsets == 1:
            p50, _ = latency_p50_us(torch, lib, fn, reps=100, warmup=10)
            res = {"p50_us": round(p50, 2)}
        else:
            _, ms = time_steps(torch, lib, fn, steps, max(3, nsets // 4))
            # a second, longer pass (about 4 ms of launches) is the one reported: a few dozen launches of a
            # kernel of a few microseconds are over before the clocks have settled, and read 30-50 % slow
            longer = min(2000, int(4.0 / ms))
            if longer > steps:
                _, ms = time_steps(torch, lib, fn, longer, max(3, nsets // 4))
            res = {"cold_gbs": round(touched / (ms * 1e-3) / 1e9, 1), "us": round(ms * 1e3, 2), "sets": nsets,
                   "launches_timed": max(longer, steps)}
        del sets
        return res

    for world in (2, 4, 8):
        row = {}
        for nbytes in sizes:
            label = f"{nbytes >> 10}KiB" if nbytes < (1 << 20) else f"{nbytes >> 20}MiB"
            row[label] = one(world, nbytes, 24 if nbytes <= (16 << 20) else 12)
            free(torch)
        out[f"w{world}"] = row
    out["config1_w8_8MiB_cold"] = one(8, 8 << 20, 36)
    free(torch)
    return out


# ------------------------------------------------------------------------------------------ other ops

MIB = 1 << 20
# bytes read and written per launch (algorithmic), for the memory-system bound of each operation
READS_WRITES = {
    "reduce_scatter_bf16": (128 * MIB, 16 * MIB), "reduce_scatter_f32": (256 * MIB, 32 * MIB),
    "all_gather_bf16": (128 * MIB, 128 * MIB), "all_gather_f32": (256 * MIB, 256 * MIB), "all_gather_int8": (64 * MIB, 64 * MIB),
    "tree_reduce_c0": (128 * MIB, 128 * MIB), "tree_reduce_c1": (256 * MIB, 128 * MIB), "tree_reduce_c2": (384 * MIB, 128 * MIB),
    "tree_copy_1": (128 * MIB, 128 * MIB), "tree_copy_2": (128 * MIB, 256 * MIB),
}


def cpu_other_ops(torch):
    """The torch CPU oracle beside two of the other operations, at their benchmark shapes: the all-gather
    pack (W rows copied into a pre-allocated [W, n]) and the tree node step with two children (fp32
    accumulate of child0, child1, own, one rounding).  Median of 5 passes after 2 warm-up passes."""
    from oracle import torch_ref
    out = {}
    n = 8_388_608
    tile = torch.randn(1 << 20, dtype=torch.bfloat16)            # values do not matter to the timing: one MiB-sized tile, repeated

    def noise_of(numel, shift):
        return tile.roll(shift).repeat(numel // tile.numel())

    # six sets of rows and outputs (1.5 GiB), one per pass: a large host's last-level cache holds one set whole
    nsets = 6
    sets = [([noise_of(n, 4099 * r + k) for r in range(WORLD)], torch.zeros((WORLD, n), dtype=torch.bfloat16))
            for k in range(nsets)]
    turn = [0]

    def gather():
        rows, packed = sets[turn[0] % nsets]
        turn[0] += 1
        for r in range(WORLD):
            packed[r].copy_(rows[r])

    def median_s(fn):
        times = []
        for i in range(7):
            t0 = time.perf_counter()
            fn()
            if i >= 2:
                times.append(time.perf_counter() - t0)
        return statistics.median(times)

    t = median_s(gather)
    assert torch.equal(sets[0][1].view(torch.int16), torch_ref.all_gather(sets[0][0]).view(torch.int16))
    out["all_gather_bf16"] = {"cpu_gbs": round(2 * WORLD * n * 2 / t / 1e9, 2), "cpu_ms": round(t * 1e3, 2)}
    del sets
    half = 67_108_864
    own, c0, c1 = (noise_of(half, 7 + 1031 * i) for i in range(3))
    t = median_s(lambda: torch_ref.tree_reduce_step(own, c0, c1))
    out["tree_reduce_c2"] = {"cpu_gbs": round(4 * half * 2 / t / 1e9, 2), "cpu_ms": round(t * 1e3, 2)}
    out["threads"] = torch.get_num_threads()
    return out


def per_process_ranks(seconds=150):
    """The collectives with every rank a process of its own on this GPU (benchlib/ipc_forms.py, 8 child
    processes started through python -m tccl_amd.launch): median us per collective of every form at 1,
    16 and 64 MiB per buffer.  A leg of its own at the very end; whatever goes wrong in it is reported,
    never raised."""
    import subprocess
    cmd = [sys.executable, "-m", "tccl_amd.launch", "--nproc-per-node", "8", "--timeout", str(seconds - 20),
           os.path.join(ROOT, "benchlib", "ipc_forms.py"), "--json", "--sizes", "1024,16384,65536"]
    try:
        done = subprocess.run(cmd, cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=seconds)
    except subprocess.TimeoutExpired:
        return {"error": f"no result within {seconds} s"}
    rows = {}
    for line in done.stdout.splitlines():
        if line.startswith('{"ipc_forms"'):
            rec = json.loads(line)
            rows[f"{rec['kib_per_buffer'] >> 10}MiB"] = rec["median_us"]
    if done.returncode != 0 or not rows:
        return {"error": f"exit code {done.returncode}: {done.stderr.strip()[-300:]}"}
    rows["note"] = ("8 processes share this GPU, one rank each; median us per collective on rank 0's stream; x3 = barrier launch + "
                    "kernel + barrier launch, fused = one launch per rank with the barriers inside the kernel")
    return rows


def other_ops(torch, tccl_amd, lib, plib, noise, device, ceilings=None):
    """The other operations of the path at their full benchmark shapes: GB/s on algorithmic bytes
    from HIP events (about 6 ms of launches after a short first pass), every one rotated over enough disjoint buffers
    that nothing is served from the 256 MB memory-side cache.  `of_bound`: the time a pure read pass
    plus a pure write pass of the same bytes would take at the cold rates measured in this run
    (cold_memory_ceilings: multi-stream read, write), divided by the operation's own time."""
    out = {}
    ops = Ops(torch, tccl_amd, lib, plib, noise, device)
    for name in ("reduce_scatter_bf16", "reduce_scatter_f32", "all_gather_bf16", "all_gather_f32", "all_gather_int8",
                 "tree_reduce_c0", "tree_reduce_c1", "tree_reduce_c2", "tree_copy_1", "tree_copy_2"):
        fn, nbytes, _ = ops.get(name)
        _, ms = time_steps(torch, lib, fn, 30, 6)
        # a second, longer pass (about 6 ms of launches) is the one reported: 36 launches of a 25 us
        # kernel right after its buffers were filled are over before the clocks have settled
        steps = min(300, max(30, int(6.0 / ms)))
        _, ms = time_steps(torch, lib, fn, steps, steps // 4)
        out[name] = {"gbs": round(nbytes / (ms * 1e-3) / 1e9, 1), "us": round(ms * 1e3, 2),
                     "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 3)}
        if ceilings and "read_8_streams_128KiB_tiles_gbs" in ceilings:
            rd, wr = READS_WRITES[name]
            bound_us = rd / ceilings["read_8_streams_128KiB_tiles_gbs"] / 1e3 + wr / ceilings["write_64MiB_32KiB_tiles_gbs"] / 1e3
            out[name]["of_bound"] = round(bound_us / (ms * 1e3), 3)
            # the same with the cost of a launch that moves almost nothing taken off the operation's time
            out[name]["of_bound_beyond_launch_cost"] = round(bound_us / (ms * 1e3 - LAUNCH_COST_US), 3)
        ops.close()
    # whole double-tree all-reduce, W=8 x 256 MiB: level schedule, pipelined single launch (both chunk sizes, both bindings)
    for how, key in (("level", "double_tree_w8_256MiB_level_schedule_ms"),
                     ("pipelined_128k", "double_tree_w8_256MiB_pipelined_128KiB_chunks_ms"),
                     ("pipelined", "double_tree_w8_256MiB_pipelined_32KiB_chunks_ms"),
                     ("pipelined_drawn", "double_tree_w8_256MiB_pipelined_drawn_places_ms")):
        fn, nbytes, _, g = ops.double_tree(how)
        _, ms = time_steps(torch, lib, fn, 5, 2)
        out[key] = round(ms, 3)
        out["double_tree_pipelined_expired_waits"] = out.get("double_tree_pipelined_expired_waits", 0) + \
            tccl_amd.signal_pad_timeouts(g)
        ops.close()
    for drawn, key in ((False, "two_shot_in_place_all_ranks_w8_64MiB_us"), (True, "two_shot_drawn_places_us")):
        fn, nbytes, _, g = ops.two_shot(drawn)
        _, ms = time_steps(torch, lib, fn, 20, 5)
        out[key] = round(ms * 1e3, 1)
        out["two_shot_expired_waits"] = out.get("two_shot_expired_waits", 0) + tccl_amd.signal_pad_timeouts(g)
        ops.close()
    return out


# ------------------------------------------------------------------------------------------ traffic evidence

def measured_traffic():
    """HBM bytes per launch of the headline kernel from the committed counter summary, and
    whether the kernel's sources are still the ones it was measured on."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None, "profiles/headline_traffic.json missing", None
    h = hashlib.sha256()
    for rel in rec.get("sources", []):
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    same = h.hexdigest()[:16] == rec.get("sources_sha256_16")
    return rec["traffic_bytes"], "profiles/headline_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, " \
        f"scaled by a 256 MiB copy: x{rec['fetch_scale']} / x{rec['write_scale']})", same


# ------------------------------------------------------------------------------------------ main

def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: W virtual ranks are W buffers on the same MI355X; "
              "runs with --gpus above 1 are not part of this build", file=sys.stderr)
        sys.exit(2)

    import torch
    import tccl_amd
    from benchlib import probe
    if args.stamps:
        # measurement build of the same sources (benchlib/stamped.hip); never the product's library
        if not args.only:
            sys.exit("--stamps needs --only OP")
        from tccl_amd import _lib
        _lib.LIB_PATH = os.path.join(ROOT, "benchlib", "libtccl_amd_stamped.so")
        _lib.SIGNATURES["tccl_stamp_buffer"] = (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_int),
                                                               ctypes.POINTER(ctypes.c_int)])
    lib = tccl_amd.load_library()
    plib = probe.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    device = "cuda:0"
    torch.cuda.set_device(0)

    if args.only:
        return run_only(args, torch, tccl_amd, lib, plib, device)

    numel = BYTES_PER_BUF // 2
    bufs_cpu = cpu_recipe(torch, WORLD, numel, torch.bfloat16)
    group = tccl_amd.empty_world(WORLD, numel, torch.bfloat16, device)
    for r in range(WORLD):
        group.tensor(r).copy_(bufs_cpu[r])
    mine = group.tensor(0)
    algo_bytes = (WORLD + 1) * numel * 2

    def step():
        return tccl_amd.one_shot_all_reduce(mine)

    for _ in range(args.preheat):
        step()
    wall_ms, dev_ms = time_steps(torch, lib, step, args.steps, args.warmup)
    gbs_wall = algo_bytes / (wall_ms * 1e-3) / 1e9
    gbs_dev = algo_bytes / (dev_ms * 1e-3) / 1e9
    noise = Noise(torch, device)         # filler for every later buffer; not needed before this point

    # The same step rotated over 8 disjoint sets of inputs AND outputs (4.6 GiB touched between
    # two uses of any byte).  On one set the 256 MB memory-side cache absorbs the 64 MiB of
    # output writes (the same output lines are rewritten every step before they are evicted)
    # and serves a little of the input; rotated like this every byte really moves over HBM.
    rot_ms = None
    try:
        extra = [make_world(tccl_amd, torch, noise, WORLD, numel, torch.bfloat16, device, salt=100 * k) for k in range(7)]
        firsts = [mine] + [g.tensor(0) for g in extra]
        outs = [torch.empty_like(mine) for _ in range(8)]
        rotated_step = Rotation(lambda k: tccl_amd.one_shot_all_reduce(firsts[k], out=outs[k]), 8)
        _, rot_ms = time_steps(torch, lib, rotated_step, max(args.steps, 40), max(args.warmup, 16))
        for g in extra:
            tccl_amd.unregister(g)
        del extra, firsts, outs, rotated_step
        free(torch)
    except RuntimeError as e:            # e.g. not enough free memory for seven more sets
        print(f"rotated measurement skipped: {e}", file=sys.stderr)

    # What the memory system gives the two halves of that launch on their own: a pure read pass
    # over the same 8 buffers and a pure write pass over one output, same launch shape.  The sum
    # is a read phase followed by a write burst, so their total is its practical bound here.
    sink = torch.zeros(4096, dtype=torch.uint8, device=device)
    probe_out = torch.empty_like(mine)
    pstream = raw_stream(torch)
    _, read_ms = time_steps(torch, lib, lambda: plib.tccl_probe_read(group.ptr_array, WORLD, BYTES_PER_BUF,
                                                                     sink.data_ptr(), pstream), 100, 50)
    _, write_ms = time_steps(torch, lib, lambda: plib.tccl_probe_write(probe_out.data_ptr(), BYTES_PER_BUF, pstream),
                             100, 50)
    ceilings = {
        "read_8x64MiB_us": round(read_ms * 1e3, 2), "read_gbs": round(WORLD * BYTES_PER_BUF / (read_ms * 1e-3) / 1e9, 1),
        "write_64MiB_us": round(write_ms * 1e3, 2), "write_gbs": round(BYTES_PER_BUF / (write_ms * 1e-3) / 1e9, 1),
        "read_pass_plus_write_pass_us": round((read_ms + write_ms) * 1e3, 2),
        "sum_kernel_us": round(dev_ms * 1e3, 2),
        "note": "the read half and the write half of the sum kernel on their own (benchlib/probe.hip), same buffers "
                "and launch shape, 100 launches each on one buffer set",
    }
    del probe_out

    # latency at 1 MiB per buffer: prefix views of the same allocations
    lat_numel = LAT_BYTES_PER_BUF // 2
    small = mine[:lat_numel]
    p50_us, p99_us = latency_p50_us(torch, lib, lambda: tccl_amd.one_shot_all_reduce(small))
    # the same launch through the C entry point alone (output allocated once, no wrapper work)
    small_out = torch.empty_like(small)
    c_call = lambda: lib.tccl_all_reduce_sum(group.ptr_array, WORLD, small_out.data_ptr(), lat_numel, 0, pstream)
    p50_c_us, _ = latency_p50_us(torch, lib, c_call)
    # what an empty kernel costs under the same event bracketing: the floor of this measurement
    floor_us, _ = latency_p50_us(torch, lib, lambda: plib.tccl_probe_empty(pstream))
    # the C entry point recorded into a HIP graph and replayed: what a caller that removes the launch path pays
    graph_us = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            lib.tccl_all_reduce_sum(group.ptr_array, WORLD, small_out.data_ptr(), lat_numel, 0, raw_stream(torch))
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            assert lib.tccl_all_reduce_sum(group.ptr_array, WORLD, small_out.data_ptr(), lat_numel, 0, raw_stream(torch)) == 0
        graph_us, _ = latency_p50_us(torch, lib, graph.replay)
        # ten replays back to back, per replay
        _, g10 = time_steps(torch, lib, graph.replay, 500, 50)
        graph_b2b_us = g10 * 1e3
        del graph
    except RuntimeError as e:
        print(f"graph replay measurement skipped: {e}", file=sys.stderr)
        graph_b2b_us = None
    # and what one wrapper call costs end to end when calls are issued back to back
    back_wall_ms, back_dev_ms = time_steps(torch, lib, lambda: tccl_amd.one_shot_all_reduce(small), 500, 50)

    cu = ctypes.c_int()
    clk = ctypes.c_int()
    bus = ctypes.c_int()
    l2 = ctypes.c_size_t()
    lib.tccl_device_info(ctypes.byref(cu), ctypes.byref(clk), ctypes.byref(bus), ctypes.byref(l2))
    traffic, traffic_source, traffic_current = measured_traffic()

    result = {
        "metric": "achieved HBM GB/s (% of 8 TB/s) W=8 bf16 reduce @64MiB/buf; p50 us @1MiB",
        "value": round(gbs_wall, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "preheat_launches": args.preheat,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",                      # the sums are accumulated in fp32 ...
        "io_dtype": "bf16",                  # ... over bf16 inputs, rounded once to a bf16 output
        "data": "synthetic: buffer r = torch.manual_seed(r); torch.randn(n, dtype=bfloat16) on the CPU, copied to its own "
                "HBM allocation before the timed region (rotated sets, other ops and the sweep: device-made N(0,1))",
        "config": {"workload": "one-shot all-reduce sum, W=8 virtual ranks, 64 MiB bf16 per buffer "
                               "(33,554,432 elements), one MI355X",
                   "world": WORLD, "bytes_per_buffer": BYTES_PER_BUF, "algorithmic_bytes_per_step": algo_bytes},
        "pct_of_peak": round(100.0 * gbs_wall / HBM_PEAK_GBS, 2),
        "rotated_over_8_buffer_sets": None if rot_ms is None else {
            "gbs": round(algo_bytes / (rot_ms * 1e-3) / 1e9, 1), "avg_launch_us": round(rot_ms * 1e3, 2),
            "frac": round(algo_bytes / (rot_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
        "memory_system_ceilings": ceilings,
        "p50_us_at_1MiB": round(p50_us, 2),
        "p99_us_at_1MiB": round(p99_us, 2),
        "p50_us_at_1MiB_c_entry_point_only": round(p50_c_us, 2),
        "launch_floor_us": round(floor_us, 2),
        "p50_us_at_1MiB_graph_replay": None if graph_us is None else round(graph_us, 2),
        "us_per_replay_at_1MiB_graph_back_to_back": None if graph_b2b_us is None else round(graph_b2b_us, 2),
        "us_per_call_at_1MiB_back_to_back": round(back_dev_ms * 1e3, 2),
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbs_dev, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs_dev / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "traffic_measured_on_these_sources": traffic_current,
            "kernel": "tccl::sum_phased_skewed_kernel<Bf16Sum, 8>",
            "avg_launch_us": round(dev_ms * 1e3, 2),
            "algorithmic_bytes": algo_bytes,
        },
        "device": {"name": torch.cuda.get_device_name(0), "compute_units": cu.value,
                   "mem_clock_khz": clk.value, "mem_bus_bits": bus.value, "l2_bytes": l2.value},
    }

    if not args.no_cpu_baseline:
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

    tccl_amd.unregister(group)
    del group, mine, small, small_out
    free(torch)

    try:
        result["cold_memory_ceilings"] = cold_ceilings(torch, lib, plib, device)
    except RuntimeError as e:
        result["cold_memory_ceilings"] = {"error": str(e)[:200]}

    if not args.no_other_ops:
        try:
            result["other_ops"] = other_ops(torch, tccl_amd, lib, plib, noise, device, result.get("cold_memory_ceilings"))
        except RuntimeError as e:        # the headline must still be printed
            result["other_ops"] = {"error": str(e)[:200]}

    if not args.no_cpu_baseline and "error" not in result.get("other_ops", {"error": 1}):
        # the CPU oracle beside the all-gather pack and the two-children tree step
        cpu = cpu_other_ops(torch)
        for name in ("all_gather_bf16", "tree_reduce_c2"):
            result["other_ops"][name].update(cpu[name])
        result["other_ops"]["cpu_threads"] = cpu["threads"]

    if not args.no_sweep:
        try:
            result["sweep"] = sweep(torch, tccl_amd, lib, noise, device)
        except RuntimeError as e:
            result["sweep"] = {"error": str(e)[:200]}

    if args.calibrate_copy:
        calibrate_copy(torch, lib, device)

    if not args.no_ipc and not args.no_other_ops:
        free(torch)
        torch.cuda.synchronize()
        result["per_process_ranks"] = per_process_ranks()

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
