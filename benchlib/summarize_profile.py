"""Short text summary of the three ``rocprofv3`` runs that profile one operation of bench.py.

    python -m benchlib.summarize_profile <dir> <op> <algorithmic read bytes> <algorithmic written bytes> [steps warmup]

<dir> holds stats/p_kernel_stats.csv (--kernel-trace --stats), fetch/p_counter_collection.csv
(--pmc FETCH_SIZE) and write/p_counter_collection.csv (--pmc WRITE_SIZE) of
``python3 bench.py --only <op>``; the two counter runs were made with --calibrate-copy, so each
holds 20 plain copies of 256 MiB whose traffic is known and scales the counter."""
from __future__ import annotations

import csv
import statistics
import sys

csv.field_size_limit(1 << 30)


def short(name: str) -> str:
    name = name.replace("void ", "").replace("tccl::", "")
    return name.split("(")[0][:90]


def counter_rows(path, counter):
    per = {}
    with open(path, newline="") as f:
        for row in csv.DictReader(f):
            if row["Counter_Name"] != counter:
                continue
            per.setdefault(short(row["Kernel_Name"]), []).append(float(row["Counter_Value"]))
    return per


def main(argv):
    d, op, rd, wr = argv[1], argv[2], int(argv[3]), int(argv[4])
    steps, warmup = (int(argv[5]), int(argv[6])) if len(argv) > 6 else (30, 6)
    print(f"Operation: bench.py --only {op}   (algorithmic bytes per launch: {rd:,} read + {wr:,} written = {rd + wr:,})")
    print("Commands (from the repository root on the GPU box, after `cd /tmp && export TMPDIR=/tmp`):")
    print(f"  rocprofv3 --kernel-trace --stats -d <dir>/stats -o p --output-format csv -- python3 bench.py --only {op} --steps {steps} --warmup {warmup}")
    print(f"  rocprofv3 --pmc FETCH_SIZE --kernel-trace -d <dir>/fetch -o p --output-format csv -- python3 bench.py --only {op} --steps 12 --warmup 4 --calibrate-copy")
    print(f"  rocprofv3 --pmc WRITE_SIZE --kernel-trace -d <dir>/write -o p --output-format csv -- python3 bench.py --only {op} --steps 12 --warmup 4 --calibrate-copy")
    print("  python -m benchlib.summarize_profile <dir> ...   (this text)")
    print()
    print(f"Kernel statistics (rocprofv3 --stats; the library's kernels only; calls = {warmup} warm-up + {steps} timed).  Which buffers a")
    print("call runs on is the operation's protocol in bench.py: the next of several disjoint buffer sets (nothing served from the")
    print("256 MB memory-side cache) for every operation except all_reduce, probe_*, two_shot* and double_tree_*, which repeat on one set:")
    print(f"  {'kernel':92s} {'calls':>5s} {'avg ns':>10s} {'min ns':>9s} {'max ns':>9s}   GB/s on algorithmic bytes")
    with open(f"{d}/stats/p_kernel_stats.csv", newline="") as f:
        for row in csv.DictReader(f):
            n = row["Name"]
            if "tccl::" not in n or "copy_kernel" in n and op != "copy_calibration":
                continue
            avg = float(row["AverageNs"])
            print(f"  {short(n):92s} {row['Calls']:>5s} {avg:10.1f} {row['MinNs']:>9s} {row['MaxNs']:>9s}   {(rd + wr) / avg:8.1f}")
    print()
    fetch = counter_rows(f"{d}/fetch/p_counter_collection.csv", "FETCH_SIZE")
    write = counter_rows(f"{d}/write/p_counter_collection.csv", "WRITE_SIZE")
    cal_f = [k for k in fetch if k.startswith("copy_kernel")]
    cal_w = [k for k in write if k.startswith("copy_kernel")]
    fs = 262144.0 / statistics.mean(fetch[cal_f[0]]) if cal_f else float("nan")
    ws = 262144.0 / statistics.mean(write[cal_w[0]]) if cal_w else float("nan")
    print("HBM traffic per launch from hardware counters (KiB per dispatch, mean over the dispatches of the counter runs):")
    print(f"  calibration: the plain copy of 256 MiB (262,144 KiB each way) reads FETCH_SIZE {statistics.mean(fetch[cal_f[0]]):,.1f}"
          f" -> x{fs:.5f}; WRITE_SIZE {statistics.mean(write[cal_w[0]]):,.1f} -> x{ws:.5f}")
    for k in sorted(set(fetch) | set(write)):
        if k.startswith("copy_kernel") or "at::native" in k or "rocclr" in k or not any(t in k for t in ("kernel<", "_kernel")):
            continue
        if not any(s in k for s in ("sum_", "pack_", "tree_", "two_shot", "probe_", "copy_")):
            continue
        f = statistics.mean(fetch.get(k, [0.0])) * fs
        w = statistics.mean(write.get(k, [0.0])) * ws
        print(f"  {k:92s} n={len(fetch.get(k, [])):3d}  fetched {f:12,.0f} KiB  written {w:12,.0f} KiB")
        print(f"  {'':92s}        = {f * 1024 / rd if rd else 0:6.4f} x algorithmic reads, {w * 1024 / wr if wr else 0:6.4f} x algorithmic writes")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
