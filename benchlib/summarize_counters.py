"""Per-channel summary of a ``rocprofv3 --pmc ... --output-format json`` run.

    python -m benchlib.summarize_counters <results.json> [kernel-name-substring]

For every kernel whose name contains the substring and every counter collected: the number of
dispatches, and over the hardware instances of the counter (for the L2's TCC counters: 16
channels x 8 XCDs = 128) the sum, the mean and the smallest and largest instance, averaged
over the dispatches -- enough to see whether a kernel loads the channels evenly."""
from __future__ import annotations

import collections
import json
import sys


def main(argv):
    path = argv[1]
    want = argv[2] if len(argv) > 2 else ""
    tool = json.load(open(path))["rocprofiler-sdk-tool"][0]
    names = {c["id"]["handle"]: c["name"] for c in tool["counters"]}
    kernels = {k["kernel_id"]: k.get("formatted_kernel_name") or k.get("demangled_kernel_name") or k["kernel_name"]
               for k in tool["kernel_symbols"]}
    # kernel -> counter -> list over dispatches of the per-instance value lists
    acc = collections.defaultdict(lambda: collections.defaultdict(list))
    times = collections.defaultdict(list)
    for rec in tool["callback_records"]["counter_collection"]:
        d = rec["dispatch_data"]
        kname = kernels.get(d["dispatch_info"]["kernel_id"], "?")
        if want not in kname:
            continue
        times[kname].append(d["end_timestamp"] - d["start_timestamp"])
        per = collections.defaultdict(list)
        for r in rec["records"]:
            per[names[r["counter_id"]["handle"]]].append(r["value"])
        for cname, vals in per.items():
            acc[kname][cname].append(vals)
    for kname, counters in acc.items():
        n = len(times[kname])
        print(f"{kname[:110]}  (dispatches: {n})")
        for cname, runs in sorted(counters.items()):
            inst = len(runs[0])
            tot = sum(sum(v) for v in runs) / len(runs)
            lo = sum(min(v) for v in runs) / len(runs)
            hi = sum(max(v) for v in runs) / len(runs)
            print(f"  {cname:34s} instances {inst:4d}  sum {tot:16,.0f}  mean {tot / inst:14,.1f}  "
                  f"min {lo:14,.1f}  max {hi:14,.1f}  max/mean {hi / (tot / inst) if tot else 0:6.3f}")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
