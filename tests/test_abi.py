"""The C-ABI library loads on a machine without a GPU, exports every symbol the header
declares, and rejects bad arguments before it would launch anything."""
import ctypes
import os
import re

import pytest

import tccl_amd
from tccl_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tccl_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tccl_[a-z0-9_]+)\s*\(", text)))


def test_header_and_loader_agree():
    syms = declared_symbols()
    assert len(syms) >= 20
    assert sorted(_lib.SIGNATURES) == syms


def test_every_declared_symbol_is_exported():
    lib = tccl_amd.load_library()
    for name in declared_symbols():
        assert getattr(lib, name) is not None, name
    assert lib.tccl_abi_version() == _lib.ABI_VERSION


def test_error_strings():
    lib = tccl_amd.load_library()
    assert lib.tccl_error_string(0) == b"ok"
    assert b"16 bytes" in lib.tccl_error_string(-2)
    assert b"power of two" in lib.tccl_error_string(-3)
    assert lib.tccl_error_string(-1001) not in (None, b"")


def test_argument_checks_return_codes_without_launching():
    """All of these return before any HIP call."""
    lib = tccl_amd.load_library()
    good = _lib.ptr_array([0x1000, 0x2000])
    odd = _lib.ptr_array([0x1000, 0x2008])
    null = _lib.ptr_array([0x1000, None])
    out = ctypes.c_void_p(0x3000)
    assert lib.tccl_all_reduce_sum(good, 0, out, 64, 0, None) == -1          # world
    assert lib.tccl_all_reduce_sum(good, 9, out, 64, 0, None) == -1
    assert lib.tccl_all_reduce_sum(good, 2, out, 64, 7, None) == -1          # dtype
    assert lib.tccl_all_reduce_sum(good, 2, None, 64, 0, None) == -1         # NULL out
    assert lib.tccl_all_reduce_sum(null, 2, out, 64, 0, None) == -1          # NULL source
    assert lib.tccl_all_reduce_sum(odd, 2, out, 64, 0, None) == -2           # alignment
    assert lib.tccl_all_reduce_sum(good, 2, ctypes.c_void_p(0x3004), 64, 0, None) == -2
    assert lib.tccl_all_reduce_sum(good, 2, out, 0, 0, None) == 0            # empty input: nothing to do
    assert lib.tccl_reduce_scatter_sum(good, 2, 2, out, 64, 0, None) == -1   # rank out of range
    assert lib.tccl_reduce_scatter_sum(good, 2, -1, out, 64, 0, None) == -1
    assert lib.tccl_reduce_scatter_sum(good, 2, 1, out, 8, 0, None) == -2    # share not 16-byte aligned ...
    assert lib.tccl_reduce_scatter_sum(good, 2, 0, out, 8, 0, None) == -2    # ... for every rank alike
    assert lib.tccl_reduce_scatter_sum(good, 2, 0, out, 17, 0, None) == -2   # not a multiple of world
    assert lib.tccl_reduce_scatter_sum(good, 2, 1, out, 4, 1, None) == -2    # fp32: a share of 2 elements is 8 bytes
    assert lib.tccl_reduce_scatter_sum(good, 2, 1, out, 0, 0, None) == 0
    assert lib.tccl_all_gather(good, 2, out, 24, None) == -2
    assert lib.tccl_all_gather(good, 0, out, 32, None) == -1
    assert lib.tccl_all_gather(good, 2, out, 0, None) == 0
    assert lib.tccl_tree_reduce_step(None, None, None, out, 64, 0, None) == -1
    assert lib.tccl_tree_reduce_step(ctypes.c_void_p(0x1008), None, None, out, 64, 0, None) == -2
    assert lib.tccl_tree_copy_step(None, out, None, 64, None) == -1
    assert lib.tccl_tree_copy_step(ctypes.c_void_p(0x1000), out, None, 24, None) == -2
    assert lib.tccl_tree_copy_step(ctypes.c_void_p(0x1000), out, None, 0, None) == 0
    assert lib.tccl_tree_level(None, 1, 0, 0, None) == -1
    assert lib.tccl_tree_level(None, 0, 9, 0, None) == -1
    assert lib.tccl_double_tree_all_reduce(good, None, 3, 64, 0, 0, None) == -3
    assert lib.tccl_double_tree_all_reduce(good, None, 128, 64, 0, 0, None) == -1
    assert lib.tccl_double_tree_all_reduce(good, None, 2, 60, 0, 0, None) == -2
    assert lib.tccl_double_tree_all_reduce(good, None, 2, 0, 0, 0, None) == 0
    assert lib.tccl_double_tree_all_reduce_fused(good, None, 16, 64, 0, None) == -1
    assert lib.tccl_double_tree_all_reduce_fused(None, None, 8, 64, 0, None) == -1
    assert lib.tccl_double_tree_all_reduce_fused(good, None, 2, 0, 0, None) == 0
    assert lib.tccl_double_tree_plan_create(good, None, 2, 64, 0, 0, None) == -1
    assert lib.tccl_plan_launch(None, None) == -1
    assert lib.tccl_plan_destroy(None) == -1
    assert lib.tccl_event_create(None) == -1
    assert lib.tccl_event_elapsed_ms(None, None, None) == -1
    # the signalling entry points
    pads = _lib.ptr_array([0x5000, 0x6000])
    sz = lib.tccl_double_tree_signal_pad_bytes
    ctl = 288 * 4                                        # control words at the end of a pad

    def rows(world):                                     # two rows of barrier slots for 512 workgroups per rank
        return 2 * 512 * world * 4

    assert sz(8, 134_217_728, 0, 65_536) == 65_536 + rows(8) + ctl       # 2 trees x 1,024 chunks x 8 flags
    assert sz(8, 134_217_728, 0, 0) == 262_144 + rows(8) + ctl           # default: 32 KiB chunks, 4,096 per tree
    assert sz(8, 134_217_728, 0, 65_536 * 2) == 32_768 + rows(8) + ctl   # 512 chunks per tree
    assert sz(2, 16, 0, 0) == 16 + rows(2) + ctl                         # one chunk per tree, two flags each
    assert sz(2, 8, 1, 0) == 16 + rows(2) + ctl
    assert sz(3, 64, 0, 0) == 0 and sz(16, 64, 0, 0) == 0 and sz(8, 60, 0, 0) == 0 and sz(8, 64, 9, 0) == 0
    piped = lib.tccl_double_tree_all_reduce_pipelined
    assert piped(good, None, pads, 16384, 3, 64, 0, 0, None, None) == -3
    assert piped(good, None, pads, 16384, 16, 64, 0, 0, None, None) == -1
    assert piped(good, None, pads, 16384, 2, 60, 0, 0, None, None) == -2
    assert piped(good, None, pads, 16384, 2, 64, 0, 12, None, None) == -2      # chunk not whole vectors
    assert piped(good, None, None, 16384, 2, 64, 0, 0, None, None) == -1
    assert piped(good, None, pads, 0, 2, 64, 0, 0, None, None) == -1          # pads too small
    assert piped(null, None, pads, 16384, 2, 64, 0, 0, None, None) == -1
    assert piped(odd, None, pads, 16384, 2, 64, 0, 0, None, None) == -2
    assert piped(good, None, pads, 16384, 2, 0, 0, 0, None, None) == 0
    ranked = lib.tccl_double_tree_all_reduce_pipelined_rank
    assert ranked(good, None, pads, 16384, 2, 2, 64, 0, 0, None, None) == -1   # rank outside the world
    assert ranked(good, None, pads, 16384, 2, -1, 64, 0, 0, None, None) == -1
    assert ranked(good, None, pads, 16384, 3, 1, 64, 0, 0, None, None) == -3
    assert ranked(good, None, pads, 16384, 2, 1, 60, 0, 0, None, None) == -2
    assert ranked(good, None, pads, 0, 2, 1, 64, 0, 0, None, None) == -1
    drawn = _lib.PipelineCfg(flags=_lib.PIPE_DRAW_PLACES)
    assert ranked(good, None, pads, 16384, 2, 1, 64, 0, 0, ctypes.byref(drawn), None) == -1   # no drawn places per rank
    assert ranked(good, None, pads, 16384, 2, 1, 0, 0, 0, None, None) == 0
    two = lib.tccl_two_shot_all_reduce
    assert two(good, None, pads, 4096, 0, 64, 0, None, None) == -1
    assert two(good, None, pads, 4096, 9, 64, 0, None, None) == -1
    assert two(good, None, pads, 4096, 2, 64, 5, None, None) == -1
    assert two(good, None, pads, 4096, 2, 24, 0, None, None) == -2            # shares not whole vectors
    assert two(good, None, pads, 1152, 2, 64, 0, None, None) == -1            # pads too small
    assert two(good, None, pads, 4090, 2, 64, 0, None, None) == -1            # pad size not a multiple of 16
    assert two(null, None, pads, 4096, 2, 64, 0, None, None) == -1
    assert two(good, None, pads, 4096, 2, 0, 0, None, None) == 0
    two_r = lib.tccl_two_shot_all_reduce_rank
    assert two_r(good, None, pads, 4096, 2, 2, 64, 0, None, None) == -1       # rank outside the world
    assert two_r(good, None, pads, 4096, 9, 0, 64, 0, None, None) == -1
    assert two_r(good, None, pads, 4096, 2, 1, 24, 0, None, None) == -2
    assert two_r(good, None, pads, 1152, 2, 1, 64, 0, None, None) == -1
    assert two_r(good, None, pads, 4096, 2, 1, 64, 0, ctypes.byref(drawn), None) == -1
    assert two_r(good, None, pads, 4096, 2, 1, 0, 0, None, None) == 0
    static = lib.tccl_two_shot_all_reduce_static
    assert static(good, None, 0, 64, 0, None, None) == -1
    assert static(good, None, 9, 64, 0, None, None) == -1
    assert static(good, None, 2, 24, 0, None, None) == -2
    assert static(null, None, 2, 64, 0, None, None) == -1
    assert static(good, None, 2, 64, 0, ctypes.byref(_lib.PipelineCfg(2 * 1024 + 1, 0, 0, 0)), None) == _lib.TCCL_ESCRATCH
    assert static(good, None, 2, 0, 0, None, None) == 0
    assert lib.tccl_timeout_flag_create(None) == -1 and lib.tccl_timeout_flag_destroy(None) == -1
    n = ctypes.c_uint(0)
    assert lib.tccl_signal_pad_timeouts(None, 4096, ctypes.byref(n), None) == -1
    assert lib.tccl_signal_pad_timeouts(ctypes.c_void_p(0x5000), 8, ctypes.byref(n), None) == -1
    assert lib.tccl_signal_pad_timeouts(ctypes.c_void_p(0x5000), 4096, None, None) == -1


def test_ipc_and_barrier_entry_points_check_their_arguments():
    lib = tccl_amd.load_library()
    pads = _lib.ptr_array([0x5000, 0x6000])
    p = ctypes.c_void_p()
    h = (ctypes.c_ubyte * _lib.IPC_HANDLE_BYTES)()
    assert lib.tccl_symm_alloc(0, ctypes.byref(p)) == -1
    assert lib.tccl_symm_alloc(1 << 31, ctypes.byref(p)) == -1          # mapped allocations stay below 2 GiB
    assert lib.tccl_symm_alloc(64, None) == -1
    assert lib.tccl_symm_free(None) == -1
    assert lib.tccl_ipc_export(None, h) == -1 and lib.tccl_ipc_open(None, ctypes.byref(p)) == -1
    assert lib.tccl_ipc_open(h, None) == -1 and lib.tccl_ipc_close(None) == -1
    bar = lib.tccl_blockwise_barrier
    assert bar(None, 4096, 2, 0, 1, 0, None, None) == -1
    assert bar(pads, 4096, 9, 0, 1, 0, None, None) == -1
    assert bar(pads, 4096, 2, 2, 1, 0, None, None) == -1
    assert bar(pads, 4096, 2, 0, 0, 0, None, None) == -1
    assert bar(pads, 4, 2, 0, 1, 0, None, None) == -1                   # pad smaller than blocks x world slots
    assert bar(_lib.ptr_array([0x5000, None]), 4096, 2, 0, 1, 0, None, None) == -1
    assert bar(_lib.ptr_array([0x5000, 0x6004]), 4096, 2, 0, 1, 0, None, None) == -2
    assert bar(pads, 4096, 1, 0, 1, 0, None, None) == 0                 # a world of one has nobody to wait for


def test_probe_library_is_separate_and_checks_its_arguments():
    """The benchmark's measuring kernels live in their own library; the product exports none of them."""
    from benchlib import probe
    plib = probe.load()
    lib = tccl_amd.load_library()
    for name in probe.SIGNATURES:
        assert not hasattr(lib, name), f"{name} is exported by the product library"
    good = _lib.ptr_array([0x1000, 0x2000])
    odd = _lib.ptr_array([0x1000, 0x2008])
    null = _lib.ptr_array([0x1000, None])
    out = ctypes.c_void_p(0x3000)
    assert plib.tccl_probe_read(good, 2, 64, None, None) == -1
    assert plib.tccl_probe_read(good, 9, 64, out, None) == -1
    assert plib.tccl_probe_read(null, 2, 64, out, None) == -1
    assert plib.tccl_probe_read(odd, 2, 64, out, None) == -2
    assert plib.tccl_probe_read(good, 2, 24, out, None) == -2
    assert plib.tccl_probe_read(good, 2, 0, out, None) == 0
    assert plib.tccl_probe_write(None, 64, None) == -1
    assert plib.tccl_probe_write(out, 24, None) == -2
    assert plib.tccl_probe_write(out, 0, None) == 0
    assert plib.tccl_probe_placement(None, 8, 0, None) == -1
    assert plib.tccl_probe_placement(out, 0, 0, None) == -1


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libtccl_amd.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()


def test_product_does_not_import_the_oracle():
    """The shipped package never reaches into oracle/."""
    pkg = os.path.join(ROOT, "tccl_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def test_struct_layouts_match_the_header(tmp_path):
    """sizeof/offsetof of the structs that cross the ABI, as gcc sees the header, against
    the ctypes mirrors."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "tccl_amd.h"\n'
        'int main(void) {\n'
        '  printf("%zu %zu %zu %zu %zu %zu\\n", sizeof(tccl_launch_cfg), offsetof(tccl_launch_cfg, block),\n'
        '         offsetof(tccl_launch_cfg, unroll), offsetof(tccl_launch_cfg, grid),\n'
        '         offsetof(tccl_launch_cfg, tile_iters), offsetof(tccl_launch_cfg, flags));\n'
        '  printf("%zu %zu %zu %zu %zu\\n", sizeof(tccl_node_job), offsetof(tccl_node_job, src),\n'
        '         offsetof(tccl_node_job, dst), offsetof(tccl_node_job, numel), offsetof(tccl_node_job, is_copy));\n'
        '  printf("%zu %zu %zu %zu %zu %zu %zu\\n", sizeof(tccl_pipeline_cfg), offsetof(tccl_pipeline_cfg, workgroups),\n'
        '         offsetof(tccl_pipeline_cfg, lag), offsetof(tccl_pipeline_cfg, spin_limit),\n'
        '         offsetof(tccl_pipeline_cfg, tile_kib), offsetof(tccl_pipeline_cfg, timeout_flag),\n'
        '         offsetof(tccl_pipeline_cfg, flags));\n'
        '  printf("%d %d %d %d %d %d\\n", TCCL_ABI_VERSION, TCCL_MAX_WORLD, TCCL_MAX_JOBS, TCCL_BF16, TCCL_F32,\n'
        '         TCCL_CFG_PHASED);\n'
        '  return 0;\n}\n')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    lines = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    cfg = [int(x) for x in lines[0].split()]
    job = [int(x) for x in lines[1].split()]
    pipe = [int(x) for x in lines[2].split()]
    consts = [int(x) for x in lines[3].split()]
    C = _lib.LaunchCfg
    assert cfg == [ctypes.sizeof(C), C.block.offset, C.unroll.offset, C.grid.offset, C.tile_iters.offset,
                   C.flags.offset]
    J = _lib.NodeJob
    assert job == [ctypes.sizeof(J), J.src.offset, J.dst.offset, J.numel.offset, J.is_copy.offset]
    P = _lib.PipelineCfg
    assert pipe == [ctypes.sizeof(P), P.workgroups.offset, P.lag.offset, P.spin_limit.offset, P.tile_kib.offset,
                    P.timeout_flag.offset, P.flags.offset]
    assert consts == [_lib.ABI_VERSION, _lib.MAX_WORLD, _lib.MAX_JOBS, _lib.TCCL_BF16, _lib.TCCL_F32,
                      _lib.CFG_PHASED]


def test_stamped_build_exports_the_same_abi_plus_its_stamp_buffer():
    """benchlib/libtccl_amd_stamped.so is the library's own sources compiled with time stamps (for
    ``bench.py --only OP --stamps``): it must export every entry point of the product, so that an
    operation runs through the same wrappers, and the product must know nothing of the stamps."""
    path = os.path.join(ROOT, "benchlib", "libtccl_amd_stamped.so")
    assert os.path.exists(path), "run python -m tccl_amd.build"
    stamped = ctypes.CDLL(path)
    for name in _lib.SIGNATURES:
        assert hasattr(stamped, name), f"{name} is missing from the stamped build"
    assert hasattr(stamped, "tccl_stamp_buffer")
    assert not hasattr(tccl_amd.load_library(), "tccl_stamp_buffer")
    stamped.tccl_stamp_buffer.restype = ctypes.c_int
    assert stamped.tccl_stamp_buffer(None, None, None) == _lib.TCCL_EINVAL


def test_per_rank_entry_points_check_their_arguments():
    """The one-shot collectives as one rank's launch: every refusal comes before anything is launched."""
    lib = tccl_amd.load_library()
    bufs = _lib.ptr_array([0x1000, 0x2000])
    pads = _lib.ptr_array([0x5000, 0x6000])
    big = 4 * (2 * 2 + 288)
    out = ctypes.c_void_p(0x3000)
    # (a launch needs a GPU: nothing here is called with arguments that would pass)
    ar, rs, ag = lib.tccl_all_reduce_sum_rank, lib.tccl_reduce_scatter_sum_rank, lib.tccl_all_gather_rank
    assert ar(None, out, pads, big, 2, 0, 64, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL
    assert ar(bufs, None, pads, big, 2, 0, 64, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL
    assert ar(bufs, out, None, big, 2, 0, 64, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL
    assert ar(bufs, out, pads, big, 2, 2, 64, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL          # rank outside the world
    assert ar(bufs, out, pads, big, 9, 0, 64, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL
    assert ar(bufs, out, pads, big - 16, 2, 0, 64, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL     # no room for two rows of slots
    assert ar(bufs, out, pads, big, 2, 0, 64, 7, None, None) == _lib.TCCL_EINVAL                       # unknown dtype
    assert ar(bufs, out, pads, big, 2, 0, 60, _lib.TCCL_BF16, None, None) == _lib.TCCL_EALIGN          # not whole vectors
    assert ar(_lib.ptr_array([0x1000, 0x2008]), out, pads, big, 2, 0, 64, _lib.TCCL_BF16, None, None) == _lib.TCCL_EALIGN
    assert ar(bufs, out, _lib.ptr_array([0x5000, 0x6004]), big, 2, 0, 64, _lib.TCCL_BF16, None, None) == _lib.TCCL_EALIGN
    drawn = _lib.PipelineCfg()
    drawn.flags = _lib.PIPE_DRAW_PLACES
    assert ar(bufs, out, pads, big, 2, 0, 64, _lib.TCCL_BF16, ctypes.byref(drawn), None) == _lib.TCCL_EINVAL
    assert rs(bufs, out, pads, big, 2, 0, 72, _lib.TCCL_BF16, None, None) == _lib.TCCL_EALIGN          # shares would be ragged
    assert rs(bufs, out, pads, big, 2, 0, 65, _lib.TCCL_BF16, None, None) == _lib.TCCL_EALIGN
    assert rs(bufs, out, pads, big, 2, 3, 64, _lib.TCCL_BF16, None, None) == _lib.TCCL_EINVAL
    assert ag(bufs, out, pads, big, 2, 0, 24, None, None) == _lib.TCCL_EALIGN
    assert ag(bufs, None, pads, big, 2, 0, 32, None, None) == _lib.TCCL_EINVAL
    # the two-shot and double-tree launches of one rank with their own barriers need more rows of slots
    own = _lib.PipelineCfg()
    own.flags = _lib.PIPE_OWN_BARRIERS
    small = 4 * (2 + 288)
    ts = lib.tccl_two_shot_all_reduce_rank
    assert ts(bufs, None, pads, small, 2, 0, 64, _lib.TCCL_BF16, ctypes.byref(own), None) == _lib.TCCL_EINVAL
    assert lib.tccl_double_tree_signal_pad_bytes(8, 1 << 20, _lib.TCCL_BF16, 0) >= 4 * (2 * 512 * 8 + 288)
