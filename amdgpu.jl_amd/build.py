"""Builds librk.so (gfx950 only) in-tree with hipcc.

    python amdgpu.jl_amd/build.py [-j N]

The element-type instantiations are separate objects (one source compiled with -DRK_INST=n) so they
build in parallel.  hipcc cross-compiles: no GPU is needed to build.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "librk.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # packed FP32 instructions are kept out of every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

# (source, object suffix, extra flags)
UNITS = (
    [("rk_api.hip", "", []), ("rk_broadcast.hip", "", []), ("rk_volumerhs.hip", "", []), ("rk_select.hip", "", []), ("rk_reverse.hip", "", []), ("rk_permute.hip", "", []), ("rk_sort.hip", "", [])]
    + [("rk_reduce_inst.hip", f"_{n}", [f"-DRK_INST={n}"]) for n in range(9)]
    + [("rk_scan_inst.hip", f"_{n}", [f"-DRK_INST={n}"]) for n in range(8)]
)


def _compile(unit):
    src, suffix, extra = unit
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + suffix + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the gfx feature flag and says so once per file: harmless
    err = "\n".join(l for l in r.stderr.splitlines() if "not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}{suffix}:\n{err}")
    return obj, err


def build(jobs: int | None = None, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(_compile, UNITS))
    for obj, err in results:
        if err.strip() and verbose:
            print(err, file=sys.stderr)
    objs = [o for o, _ in results]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    if verbose:
        print(f"built {LIB} ({os.path.getsize(LIB) >> 10} KiB) from {len(objs)} objects")
    return LIB


if __name__ == "__main__":
    j = None
    if "-j" in sys.argv:
        j = int(sys.argv[sys.argv.index("-j") + 1])
    build(j)
