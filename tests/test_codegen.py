"""What hipcc makes of the kernels, checked on the assembly it emits for gfx950 (no GPU
needed): no packed fp32 arithmetic, no scratch memory, no scalar-cache writes, and the
phased sum kernel small enough for two workgroups per compute unit."""
import os
import re
import shutil
import subprocess

import pytest

from tccl_amd import build as lib_build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"),
                                reason="hipcc not available")


@pytest.fixture(scope="module", params=lib_build.SOURCES)
def asm(request, tmp_path_factory):
    src = os.path.join(ROOT, "tccl_amd", "csrc", request.param)
    out = tmp_path_factory.mktemp("asm") / (request.param + ".s")
    flags = [f for f in lib_build.HIPCC_FLAGS if f != "-fPIC"]
    cmd = [lib_build._hipcc(), *flags, "-S", "--cuda-device-only", src, "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    return request.param, out.read_text()


def test_no_packed_fp32_no_scratch_no_scalar_stores(asm):
    name, text = asm
    assert not re.search(r"\bv_pk_(add|mul|fma)_f32\b", text), f"{name}: packed fp32 arithmetic"
    assert not re.search(r"\b(s_store_dword|s_buffer_store|s_dcache_wb|s_dcache_inv|s_atomic_)", text), name
    sizes = [int(m) for m in re.findall(r"\.private_segment_fixed_size:\s*(\d+)", text)]
    assert all(s == 0 for s in sizes), f"{name}: a kernel uses scratch memory"
    if name != "util.hip":                 # util.hip is host code only
        assert sizes and ".wavefront_size: 64" in text


def test_phased_kernels_fit_two_workgroups_per_cu(asm):
    name, text = asm
    if name != "sum.hip":
        pytest.skip("only the sum kernels")
    # every kernel record: name ... vgpr_count
    records = re.findall(r"\.name:\s+(\S*sum_phased_(?:skewed_)?kernel\S*)\n(?:.*\n)*?\s+\.vgpr_count:\s+(\d+)", text)
    assert len(records) >= 40 and any("skewed" in k for k, _ in records)
    for kernel, vgprs in records:
        # 256 lanes = one wave per SIMD per workgroup; two workgroups need <= 256 VGPRs each
        assert int(vgprs) <= 256, (kernel, vgprs)
    w8 = [int(v) for k, v in records if "Bf16SumELi8ELi1ELb1" in k]
    assert w8 and w8[0] <= 256
    assert "v_cvt_pk_bf16_f32" in text and "buffer_load_dwordx4" in text and "buffer_store_dwordx4" in text


def test_pipelined_kernel_uses_device_scope_accesses_and_no_cache_flushes(asm):
    """The pipelined double tree keeps its workgroups coherent across the XCDs' L2 caches with
    device-scope (sc1) loads and stores alone; a whole-cache write-back or invalidate per
    signal would cost more than the chunk it guards."""
    name, text = asm
    if name != "pipeline.hip":
        pytest.skip("only the pipelined kernel")
    # function bodies by kernel name: from "<mangled name>:" to the function's end label
    bodies = dict(re.findall(r"^(_ZN4tccl\S+):[^\n]*\n(.*?)^\.Lfunc_end", text, flags=re.S | re.M))
    tree = [b for n, b in bodies.items() if "tree_pipelined_kernel" in n]
    two_shot = [b for n, b in bodies.items() if "two_shot_kernel" in n]
    assert len(tree) == 4 and len(two_shot) == 16
    for body in tree + two_shot:
        # The place a workgroup draws at run time must reach the data path as a wave-uniform
        # value: if it does not, every buffer access is wrapped in a loop over the distinct
        # descriptors of the lanes (dozens of v_readfirstlane per access, +15 % run time).
        assert body.count("v_readfirstlane_b32") < 64, "buffer descriptors are not wave-uniform"
        loads = re.findall(r"buffer_load_dwordx4[^\n]*", body)
        stores = re.findall(r"buffer_store_dwordx4[^\n]*", body)
        assert loads and stores
        assert all(re.search(r"\bsc1\b", line) for line in stores), "a data store is not device-scope"
        flags = re.findall(r"global_(?:load|store)_dword [^\n]*", body)
        if body in tree:
            # every source may have been rewritten by a peer during the kernel
            assert all(re.search(r"\bsc1\b", line) for line in loads), "a data load is not device-scope"
        assert all(re.search(r"\bsc1\b", line) for line in flags), "a flag access is not device-scope"
    # two-shot: the first shot reads the call's inputs (streaming loads), the second shot reads
    # what peers wrote during the kernel (device-scope loads)
    w8 = [b for n, b in bodies.items() if "two_shot_kernel" in n and "Li8E" in n][0]
    loads = re.findall(r"buffer_load_dwordx4[^\n]*", w8)
    assert any(not re.search(r"\bsc1\b", line) for line in loads) and any(re.search(r"\bsc1\b", line) for line in loads)
    assert "buffer_wbl2" not in text and "buffer_inv" not in text
    assert "s_sleep" in text and "global_atomic_add" in text
    # No signalling grid may reach 8 workgroups (32 waves) per compute unit, the one shape that once timed
    # out for an unknown reason.  Some kernels are small enough for it by their registers (512 per SIMD lane,
    # 8 per allocation: the two-shot kernel for a world of three needs 62), so the launcher's cap is what
    # keeps it away: every launch site asks resident_for, and resident_for cuts at 6.
    small = [n for n, v in re.findall(r"\.name:\s+(\S*(?:tree_pipelined_kernel|two_shot_kernel|two_shot_rank_kernel|_rank_kernel)\S*)\n(?:.*\n)*?\s+\.vgpr_count:\s+(\d+)", text)
             if 512 // ((int(v) + 7) // 8 * 8) > 6]
    assert small, "the cap has become unreachable: say so here"
    source = open(os.path.join(ROOT, "tccl_amd", "csrc", "pipeline.hip")).read()
    assert "constexpr int kMaxSignallingPerUnit = 6;" in source
    assert "if (per_cu > kMaxSignallingPerUnit) per_cu = kMaxSignallingPerUnit;" in source
    assert source.count("hipOccupancyMaxActiveBlocksPerMultiprocessor(") == 1      # resident_for is the only one who asks
    # One launch per rank (the peers are other processes' kernels, which may start and end at any time):
    # every data load is device-scope, shot 1 of the two-shot kernel included; flags are raised by
    # device-scope stores and taken by device-scope compare-and-swaps.
    per_rank = {n: b for n, b in bodies.items() if any(k in n for k in ("sum_rank_kernel", "gather_rank_kernel",
                                                                        "two_shot_rank_kernel"))}
    assert len(per_rank) == 16 + 1 + 16
    for n, body in per_rank.items():
        loads = re.findall(r"buffer_load_dwordx4[^\n]*", body)
        stores = re.findall(r"buffer_store_dwordx4[^\n]*", body)
        assert loads and stores, n
        assert all(re.search(r"\bsc1\b", line) for line in loads), f"{n}: a data load is not device-scope"
        assert all(re.search(r"\bsc1\b", line) for line in stores), f"{n}: a data store is not device-scope"
        if "Li1E" in n and "gather" not in n:
            continue                          # a world of one has nobody to wait for
        swaps = re.findall(r"global_atomic_cmpswap[^\n]*", body)
        raises = re.findall(r"global_store_dword [^\n]*", body)
        assert swaps, f"{n}: flags are not taken with compare-and-swap"     # (a read-modify-write is carried out beyond the XCD's L2 as it is)
        assert raises and all(re.search(r"\bsc1\b", line) for line in raises), f"{n}: flags are not raised at device scope"
        assert body.count("v_readfirstlane_b32") < 64, f"{n}: buffer descriptors are not wave-uniform"
