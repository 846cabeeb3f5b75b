"""Start a per-rank program once per rank on ONE GPU, the way the reference's programs are started
by torchrun (triton_one_shot_all_reduce_no_128.py:99-110 reads RANK, LOCAL_RANK and WORLD_SIZE):

    python -m tccl_amd.launch --nproc-per-node 8 program.py [arguments of the program ...]
    python -m tccl_amd.launch --nproc-per-node 8 --module tccl_amd.harness all_reduce [...]

Every rank is a process of its own with RANK = 0 .. W-1, WORLD_SIZE = W, LOCAL_RANK = 0 (all ranks
share the one GPU) and TCCL_RENDEZVOUS_DIR = a fresh directory through which the ranks exchange
their buffer handles; ``tccl_amd.ipc.IpcWorld.from_env()`` in the program picks these up.  The
launcher itself never touches the GPU.  Its exit code is the exit code of the first rank that
failed (124 if the time limit ended the run).  When a rank fails, its peers would wait for it in the
next rendezvous or barrier until their own bounded waits expire: they get ``--grace`` seconds to
end by themselves and are stopped then, and so is every rank still running at ``--timeout``."""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
import tempfile
import time


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m tccl_amd.launch", description=__doc__.split("\n\n")[0])
    ap.add_argument("--nproc-per-node", type=int, required=True, help="ranks (processes) to start, 1..8")
    ap.add_argument("--timeout", type=float, default=600.0, help="seconds before ranks still running are stopped")
    ap.add_argument("--grace", type=float, default=10.0, help="seconds the other ranks may run on after one has failed")
    ap.add_argument("--module", help="run this module once per rank (python -m MODULE) instead of a program file")
    ap.add_argument("program", nargs="?", help="the per-rank program (a Python file)")
    ap.add_argument("args", nargs=argparse.REMAINDER, help="its arguments")
    ns = ap.parse_args(argv)
    if not 1 <= ns.nproc_per_node <= 8:
        ap.error("--nproc-per-node must be 1..8")
    if ns.module:                        # what argparse took for the program is the module's first argument
        command = [sys.executable, "-m", ns.module] + ([ns.program] if ns.program else []) + ns.args
    elif ns.program:
        command = [sys.executable, ns.program, *ns.args]
    else:
        ap.error("a program file or --module is needed")
    directory = tempfile.mkdtemp(prefix="tccl_rendezvous_")
    procs = []
    try:
        for rank in range(ns.nproc_per_node):
            env = dict(os.environ, RANK=str(rank), LOCAL_RANK="0", WORLD_SIZE=str(ns.nproc_per_node),
                       TCCL_RENDEZVOUS_DIR=directory)
            procs.append(subprocess.Popen(command, env=env))
        code = 0
        deadline = time.monotonic() + ns.timeout
        running = list(procs)
        while running:
            for p in list(running):
                rc = p.poll()
                if rc is None:
                    continue
                running.remove(p)
                if rc != 0 and code == 0:            # the first failure: the others' time is limited from now on
                    code = rc
                    deadline = min(deadline, time.monotonic() + ns.grace)
            if running and time.monotonic() >= deadline:
                if code == 0:
                    code = 124
                break                                # what still runs is stopped below
            if running:
                time.sleep(0.05)
        return code
    finally:
        for p in procs:                      # exactly the processes started here
            if p.poll() is None:
                p.kill()
                p.wait()
        shutil.rmtree(directory, ignore_errors=True)


if __name__ == "__main__":
    sys.exit(main())
