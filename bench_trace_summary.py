#!/usr/bin/env python3
"""Per-row kernel summary of a `rocprofv3 --kernel-trace --marker-trace` run of bench.py.

    rocprofv3 --kernel-trace --marker-trace --output-format csv -d DIR -o bench -- python3 bench.py --no-cpu
    python bench_trace_summary.py DIR/bench > profiles/<name>.txt

bench.py runs every row of its table inside a roctx range named like the row.  This script assigns each kernel
dispatch of the trace to the range it started in and prints, per row, the kernels it launched: calls, average /
minimum / maximum duration, grid and workgroup size, registers.  Each range holds the row's warm-up launches, its
individually synchronised launches and its back-to-back launches, so `avg` mixes the two timing modes; `min` is the
figure to compare with the row's `min_us` (which adds the launch and event overhead seen from the host).
"""
from __future__ import annotations

import csv
import re
import sys
from collections import OrderedDict, defaultdict


def short(name: str, limit: int = 110) -> str:
    name = re.sub(r"^void ", "", name)
    name = name.replace("rk::", "")
    name = re.sub(r"\(.*\)$", "", name)          # argument list
    return name if len(name) <= limit else name[:limit - 3] + "..."


def main():
    if len(sys.argv) != 2:
        sys.exit(__doc__)
    base = sys.argv[1]
    ranges = []
    with open(base + "_marker_api_trace.csv", newline="") as fh:
        for r in csv.DictReader(fh):
            ranges.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), r["Function"]))
    ranges.sort()
    rows = OrderedDict((name, defaultdict(list)) for _, _, name in ranges)
    outside = 0
    with open(base + "_kernel_trace.csv", newline="") as fh:
        for r in csv.DictReader(fh):
            t0, t1 = int(r["Start_Timestamp"]), int(r["End_Timestamp"])
            if "at::native" in r["Kernel_Name"] or r["Kernel_Name"].startswith("__amd_rocclr"):
                outside += 1                      # torch's own kernels (input generation, refills): not the library's
                continue
            hit = None
            for a, b, name in ranges:
                if a <= t0 <= b:
                    hit = name
                    break
            if hit is None:
                outside += 1
                continue
            key = (short(r["Kernel_Name"]), f'{r["Grid_Size_X"]}x{r["Grid_Size_Y"]}x{r["Grid_Size_Z"]}',
                   f'{r["Workgroup_Size_X"]}x{r["Workgroup_Size_Y"]}x{r["Workgroup_Size_Z"]}', r["VGPR_Count"], r["LDS_Block_Size"])
            rows[hit][key].append((t1 - t0) / 1e3)
    print("# kernels per bench row: calls, avg / min / max duration in us, grid (work-items), workgroup, VGPRs, LDS bytes")
    print(f"# ({outside} dispatches left out: outside any row, or torch's / the runtime's own kernels -- input generation, refills, clears)")
    for name, kernels in rows.items():
        print(f"\n== {name}")
        for (kname, grid, wg, vgpr, lds), d in sorted(kernels.items(), key=lambda kv: -sum(kv[1])):
            print(f"   {len(d):4d} x  avg {sum(d) / len(d):9.2f}  min {min(d):9.2f}  max {max(d):9.2f}   grid {grid:>16s}  wg {wg:>9s}  vgpr {vgpr:>3s}  lds {lds:>6s}   {kname}")


if __name__ == "__main__":
    main()
