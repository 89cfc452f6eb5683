#!/usr/bin/env python3
"""HBM traffic per kernel from two rocprofv3 counter runs of bench.py (FETCH_SIZE, then WRITE_SIZE).

    ONLY='sum Float32[2^26]|maximum|cumsum Int32[2^26]|z .= a.*x .+ y.*exp.(w) Float32[2^26]|calibration: copy z .= x Float32[2^26]|cfg2|cfg3|cumsum(B;dims=2)|cfg4|cfg5|Int16|Float16|Float64|sum(A; dims=|cumsum(A; dims=1) 15x|C .= A .+ r 3x|permutedims|reverse|findall'
    rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d F -o bench -- python3 bench.py --no-cpu --steps 5 --only "$ONLY"
    rocprofv3 --pmc WRITE_SIZE --kernel-trace --output-format csv -d W -o bench -- python3 bench.py --no-cpu --steps 5 --only "$ONLY"
    python bench_pmc_summary.py F/bench W/bench > profiles/<name>.txt

The counters are KiB per dispatch in units the hardware defines; they are scaled by what the same counter reads for
the plain copy kernel of known size in the same run (z .= x on 2^26 Float32: 262144 KiB read, 262144 KiB written).
Rows are kernel x grid, averaged over the dispatches of the run; `alg` is the algorithmic traffic of that launch
where this script knows the row (the sizes of bench.py's configurations)."""
from __future__ import annotations

import csv
import re
import sys
from collections import defaultdict

KIB = 1024.0
# (kernel-name fragment, grid work-items) -> (row of bench.py, algorithmic KiB read, written)
M26, M27 = (1 << 26), (1 << 27)
N25 = 1 << 25
N15, N3 = (N25 // 15) * 15, (N25 // 3) * 3
KNOWN = [
    ("bc_flat_kernel<EvalCopy", 16777216, "calibration: copy z .= x Float32[2^26]", 4 * M26 / KIB, 4 * M26 / KIB),
    ("bc_flat_kernel<EvalAxpbyExp", 16777216, "z .= a.*x .+ y.*exp.(w) Float32[2^26]", 12 * M26 / KIB, 4 * M26 / KIB),
    ("bc_flat_kernel<EvalAxpbyExp", 33554432, "cfg4a z .= a.*x .+ y.*exp.(w) 512^3", 12 * M27 / KIB, 4 * M27 / KIB),
    ("bc_kernel<EvalAddMul", None, "cfg4b C .= A .+ r .* c 16384^2", 4 * (1 << 28) / KIB, 4 * (1 << 28) / KIB),
    ("scan_ordered_kernel<int", 2097152, "cumsum Int32[2^26]", 4 * M26 / KIB, 4 * M26 / KIB),
    ("scan_ordered_kernel<int", 4194304, "cfg3a cumsum Int32[2^27]", 4 * M27 / KIB, 4 * M27 / KIB),
    ("scan_ordered_kernel<short", None, "cumsum Int16[2^26] (native narrow scan, 4 B/elt)", 2 * M26 / KIB, 2 * M26 / KIB),
    ("bc_kernel<EvalChain2, float, 8", None, "z .= a.*x .+ y Float16[2^26] (6 B/elt)", 4 * M26 / KIB, 2 * M26 / KIB),
    ("bc_flat_kernel<EvalChain2, double", None, "z .= a.*x .+ y Float64[2^26] (24 B/elt)", 16 * M26 / KIB, 8 * M26 / KIB),
    ("scan_tiles_kernel<float", None, "cfg3b cumsum(B;dims=1) 4096x16384", 4 * M26 / KIB, 4 * M26 / KIB),
    ("scan_tiles_kernelIDF16_", None, "cumsum(B;dims=1) 4096x16384 Float16 (native narrow scan, 4 B/elt)", 2 * M26 / KIB, 2 * M26 / KIB),   # (left mangled by the profiler)
    ("scan_tiles_kernel<_Float16", None, "cumsum(B;dims=1) 4096x16384 Float16 (native narrow scan, 4 B/elt)", 2 * M26 / KIB, 2 * M26 / KIB),
    ("scan_rows_ordered_kernel<float", None, "cumsum(B;dims=2) 4096x16384", 4 * M26 / KIB, 4 * M26 / KIB),
    ("MapIdentity>, OpAdd, ReduceSink<float, OpAdd, float>, true", 131072, "sum Float32 (2^26: 262144 KiB; the 2^24 row shares this grid)", None, None),
    ("MapIdentity>, OpMax", 131072, "maximum Float32[2^26]", 4 * M26 / KIB, 0.0),
    ("MapAbs2>, OpAdd", None, "cfg2a / cfg2b mapreduce(abs2,+) 8192^2", 4 * M26 / KIB, 32.0),
    ("ArgXform<float", None, "cfg2c findmax(A;dims=1) 8192^2", 4 * M26 / KIB, 160.0),
    ("volumerhs_vec_kernel", None, "cfg5 volumerhs! nelem=240000", 240000 * 11000 / KIB, 240000 * 2500 / KIB),
    ("volumerhs_kernel", None, "cfg5 volumerhs! nelem=4000", 4000 * 11000 / KIB, 4000 * 2500 / KIB),
    # shapes with short or narrow extents, 2^25 elements (the rows bench.py keeps below the benchmark configurations)
    ("reduce_short_lines_kernel", None, "sum(A; dims=1) 32x1048576 / sum(A; dims=2) 4x32x262144", 4 * N25 / KIB, 4 * (N25 // 32) / KIB),
    ("scan_lds_lines_kernel<float", None, "cumsum(A; dims=1) 15x2236962", 4 * N15 / KIB, 4 * N15 / KIB),
    ("bc_indexed_kernel<EvalBinary", None, "C .= A .+ r 3x11184810 .+ 1x11184810", (4 * N3 + 4 * (N3 // 3)) / KIB, 4 * N3 / KIB),
    ("permute_slab_kernel", None, "permutedims(A, (3,2,1)) 2x8388608x2", 4 * N25 / KIB, 4 * N25 / KIB),
    ("permute_tiles_vec_kernel", None, "permutedims(A, (2,1)) 8192^2", 4 * M26 / KIB, 4 * M26 / KIB),
    ("reverse_kernel", None, "reverse(A; dims=1) 8192^2", 4 * M26 / KIB, 4 * M26 / KIB),
    ("findall_select_kernel", None, "findall(Bool[2^26], 25 % true): 1 B/elt read, 8 B per index written", M26 / KIB, 8 * 0.25 * M26 / KIB),
]


def short(name: str, limit: int = 84) -> str:
    name = re.sub(r"^void ", "", name).replace("rk::", "")
    name = re.sub(r"\(.*\)$", "", name)
    return name if len(name) <= limit else name[:limit - 3] + "..."


def load(base, counter):
    acc = defaultdict(list)
    with open(base + "_counter_collection.csv", newline="") as fh:
        for r in csv.DictReader(fh):
            if r["Counter_Name"] != counter or "at::native" in r["Kernel_Name"]:
                continue
            acc[(short(r["Kernel_Name"]), int(r["Grid_Size"]))].append(float(r["Counter_Value"]))
    return {k: sum(v) / len(v) for k, v in acc.items()}, {k: len(v) for k, v in acc.items()}


def main():
    if len(sys.argv) != 3:
        sys.exit(__doc__)
    fetch, nf = load(sys.argv[1], "FETCH_SIZE")
    write, _ = load(sys.argv[2], "WRITE_SIZE")
    cal = [k for k in fetch if k[0].startswith("bc_flat_kernel<EvalCopy") and k[1] == 16777216]
    if not cal:
        sys.exit("the calibration kernel (copy of 2^26 Float32) is not in the run")
    ff = 262144.0 / fetch[cal[0]]
    fw = 262144.0 / write[cal[0]]
    print(f"# calibration on {cal[0][0]}: FETCH_SIZE x {ff:.4f}, WRITE_SIZE x {fw:.4f}")
    print(f"# {'kernel':84s} {'grid':>10s} {'calls':>5s} {'read KiB':>10s} {'write KiB':>10s} {'alg read':>10s} {'alg write':>10s} {'traffic/alg':>11s}  row")
    for k in sorted(fetch, key=lambda k: (k[0], k[1])):
        rd, wr = fetch[k] * ff, write.get(k, 0.0) * fw
        row, ar, aw = "", None, None
        for frag, grid, name, r_, w_ in KNOWN:
            if frag in k[0] and (grid is None or grid == k[1]):
                row, ar, aw = name, r_, w_
                break
        ratio = f"{(rd + wr) / (ar + aw):11.4f}" if ar is not None else " " * 11
        print(f"  {k[0]:84s} {k[1]:10d} {nf[k]:5d} {rd:10.0f} {wr:10.0f} {ar if ar is not None else float('nan'):10.0f} {aw if aw is not None else float('nan'):10.0f} {ratio}  {row}")


if __name__ == "__main__":
    main()
