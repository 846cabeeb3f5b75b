"""Build recipe for ``libtccl_amd.so`` (hipcc, gfx950 only).

``python -m tccl_amd.build`` compiles every ``csrc/*.hip`` into an object file and links
the shared library next to this file.  The library is built in-tree so that it travels
with the source tree; nothing is compiled at import time.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from typing import List

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "_obj")
LIB_PATH = os.path.join(HERE, "libtccl_amd.so")

SOURCES = ["sum.hip", "gather.hip", "tree.hip", "pipeline.hip", "ipc.hip", "util.hip"]

# -ffp-contract=off: the sums are adds only, but nothing may ever be fused.
# -packed-fp32-ops off: keep the compiler from forming v_pk_add_f32 out of the
# accumulator adds; each add stays a scalar v_add_f32.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libtccl_amd.so can only be built with ROCm's hipcc")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    return obj


def build(verbose: bool = False, jobs: int = 4) -> str:
    """Compile and link the library; returns its path.  Always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs: List[str] = list(pool.map(_compile, SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH)} bytes)")
    return LIB_PATH


def build_probe(verbose: bool = False) -> str:
    """Compile the benchmark's measuring kernels (benchlib/probe.hip) into their own library,
    benchlib/libtccl_probe.so: they are loaded by bench.py only and are no part of the product."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "benchlib", "probe.hip")
    out = os.path.join(root, "benchlib", "libtccl_probe.so")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-shared", src, "-o", out + ".tmp"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on probe.hip:\n{proc.stdout}\n{proc.stderr}")
    os.replace(out + ".tmp", out)
    if verbose:
        print(f"built {out}")
    return out


def build_stamped(verbose: bool = False) -> str:
    """Compile the measurement build of the library (benchlib/stamped.hip: every csrc/*.hip as one
    translation unit with TCCL_STAMPS defined) into benchlib/libtccl_amd_stamped.so.  Loaded by
    ``bench.py --only OP --stamps`` only; no part of the product."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "benchlib", "stamped.hip")
    out = os.path.join(root, "benchlib", "libtccl_amd_stamped.so")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-shared", src, "-o", out + ".tmp"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on stamped.hip:\n{proc.stdout}\n{proc.stderr}")
    os.replace(out + ".tmp", out)
    if verbose:
        print(f"built {out}")
    return out


def build_c_client(verbose: bool = False) -> str:
    """Compile the plain C client of the library (tests/c_client) next to its source."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "c_client", "c_abi_client.c")
    out_dir = os.path.join(root, "tests", "c_client", "build")
    os.makedirs(out_dir, exist_ok=True)
    exe = os.path.join(out_dir, "c_abi_client")
    cmd = [_hipcc(), "-x", "c", "-std=c11", "-O1", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(root, "include"),
           "-I", "/opt/rocm/include", src, "-L", HERE, "-ltccl_amd", "-L", "/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath," + HERE, "-Wl,-rpath,/opt/rocm/lib", "-o", exe]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building the C client failed:\n{proc.stdout}\n{proc.stderr}")
    if verbose:
        print(f"built {exe}")
    return exe


if __name__ == "__main__":
    build(verbose=True)
    build_probe(verbose=True)
    build_stamped(verbose=True)
    build_c_client(verbose=True)
    sys.exit(0)
