"""Builds librk.so (gfx950 only) in-tree with hipcc.

    python amdgpu.jl_amd/build.py [-j N] [--incremental]

The element-type instantiations are separate objects (one source compiled with -DRK_INST=n) so they
build in parallel.  hipcc cross-compiles: no GPU is needed to build.
"""
from __future__ import annotations

import hashlib
import os
import re
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
    # per-kernel register / private-memory report of the device pass, checked below
    "-Rpass-analysis=kernel-resource-usage",
]

# (source, object suffix, extra flags)
UNITS = (
    [("rk_api.hip", "", []), ("rk_broadcast.hip", "", []), *[("rk_broadcast.hip", f"_{n}", [f"-DRK_BC_INST={n}"]) for n in range(6)], ("rk_volumerhs.hip", "", []), ("rk_select.hip", "", []), ("rk_reverse.hip", "", []), ("rk_permute.hip", "", []), ("rk_sort.hip", "", [])]
    + [("rk_reduce_inst.hip", f"_{n}", [f"-DRK_INST={n}"]) for n in range(13)]
    + [("rk_scan_inst.hip", f"_{n}", [f"-DRK_INST={n}"]) for n in range(13)]
)


def _stamp_path(unit) -> str:
    src, suffix, _ = unit
    return os.path.join(OBJ, os.path.splitext(src)[0] + suffix + ".stamp")


def _flags_key(unit) -> str:
    """What the object depends on besides its sources: the compiler and every flag of the unit."""
    return hashlib.sha256("\0".join([HIPCC, *FLAGS, *unit[2]]).encode()).hexdigest()


def _compile(unit):
    src, suffix, extra = unit
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + suffix + ".o")
    stamp = _stamp_path(unit)
    if os.path.exists(stamp):
        os.remove(stamp)                 # no stamp = not a checked object: an interrupted or failed build leaves none
    cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # No kernel of this library may keep an array in private memory: the ones that did (operand registers indexed with a
    # computed address, a tile the optimizer failed to split into registers) ran 1.8-16x slower.  The report of the
    # device pass gives private bytes per lane and spilled registers; a few spilled registers at the 128-register cap
    # of the 1024-thread kernels are tolerated, anything beyond them is not.
    private, lines, skip = [], [], 0
    cur = {}

    def close():
        if cur and cur.get("scratch", 0) > 4 * cur.get("vspill", 0) + 8 or cur.get("vspill", 0) > 16:
            private.append(f"{cur['name']}: {cur['scratch']} bytes of private memory per lane, {cur.get('vspill', 0)} spilled registers")
    pending = []                     # "In file included from" lines belong to the diagnostic that follows them
    for l in r.stderr.splitlines():
        if l.startswith("In file included from"):
            pending.append(l)
            continue
        if "-Rpass-analysis=kernel-resource-usage" in l:
            pending = []
            m = re.search(r"remark:\s+Function Name: (\S+)", l)
            if m:
                close()
                cur = {"name": m.group(1)}
            m = re.search(r"remark:\s+ScratchSize \[bytes/lane\]: (\d+)", l)
            if m:
                cur["scratch"] = int(m.group(1))
            m = re.search(r"remark:\s+VGPRs Spill: (\d+)", l)
            if m:
                cur["vspill"] = int(m.group(1))
            skip = 2 if "Function Name" in l else 0      # the remark's source line and caret follow
            continue
        if skip > 0:
            skip -= 1
            continue
        # the host pass does not know the gfx feature flag and says so once per file: harmless
        if "not a recognized feature" not in l:
            lines.extend(pending)
            lines.append(l)
        pending = []
    close()
    err = "\n".join(lines)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}{suffix}:\n{err}")
    if not private:
        # the stamp records the flags the object was built with and that it passed the private-memory check; an
        # incremental build recompiles every unit whose stamp is missing or was written for other flags
        with open(stamp, "w") as f:
            f.write(_flags_key(unit) + "\n")
    return obj, err, [f"{src}{suffix}: {p}" for p in private]


def _stale(unit) -> bool:
    """True when the unit's object is older than its source or any header of the library, was built with other
    flags, or did not pass the private-memory check (no stamp)."""
    src, suffix, _ = unit
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + suffix + ".o")
    stamp = _stamp_path(unit)
    if not os.path.exists(obj) or not os.path.exists(stamp) or open(stamp).read().strip() != _flags_key(unit):
        return True
    t = os.path.getmtime(obj)
    deps = [os.path.join(CSRC, src), os.path.join(HERE, "..", "include", "rk.h")]
    text = open(os.path.join(CSRC, src)).read()
    seen, todo = set(), re.findall(r'#include "([^"]+)"', text)
    while todo:                                   # headers of csrc/, transitively
        h = os.path.basename(todo.pop())
        if h in seen or not os.path.exists(os.path.join(CSRC, h)):
            continue
        seen.add(h)
        deps.append(os.path.join(CSRC, h))
        todo += re.findall(r'#include "([^"]+)"', open(os.path.join(CSRC, h)).read())
    return any(os.path.getmtime(d) > t for d in deps)


def build(jobs: int | None = None, verbose: bool = True, incremental: bool = False) -> str:
    """Compile and link.  ``incremental`` recompiles only the units whose sources or flags changed; every linked object
    carries a stamp saying that it passed the private-memory check with the current flags."""
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    units = [u for u in UNITS if _stale(u)] if incremental else list(UNITS)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(_compile, units))
    for obj, err, _ in results:
        if err.strip() and verbose:
            print(err, file=sys.stderr)
    private = [p for _, _, ps in results for p in ps]
    if private:
        raise RuntimeError("kernels using private memory:\n  " + "\n  ".join(private))
    objs = [os.path.join(OBJ, os.path.splitext(src)[0] + suffix + ".o") for src, suffix, _ in UNITS]
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
    build(j, incremental="--incremental" in sys.argv)
