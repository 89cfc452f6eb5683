"""Host mirror of the ``@roc ... volumerhs!(rhs, Q, vgeo, gravity, D, nelem)`` call site
(perf/volumerhs.jl:200-201).  N = 4 is fixed like the reference's benchmark (perf/volumerhs.jl:35)."""
from __future__ import annotations

import numpy as np

from . import _lib as L
from .array import ROCArray, stream_ptr

NQ, NSTATE, NVGEO = 5, 5, 14
GRAV = 9.81          # perf/volumerhs.jl:39


def volumerhs_(rhs: ROCArray, Q: ROCArray, vgeo: ROCArray, gravity, D: ROCArray, nelem: int) -> ROCArray:
    """Accumulates the DG volume terms of the Euler equations into ``rhs`` (in place) and returns it.

    rhs, Q: (5,5,5,5,nelem); vgeo: (5,5,5,14,nelem); D: (5,5); all Float32, column-major."""
    nelem = int(nelem)
    want = {"rhs": (rhs, (NQ, NQ, NQ, NSTATE, nelem)), "Q": (Q, (NQ, NQ, NQ, NSTATE, nelem)),
            "vgeo": (vgeo, (NQ, NQ, NQ, NVGEO, nelem)), "D": (D, (NQ, NQ))}
    for name, (arr, dims) in want.items():
        if arr.dtype != np.float32:
            raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"volumerhs!: {name} must be Float32")
        if arr.dims != dims:
            raise L.DimensionMismatch(L.RK_ERR_DIMENSION, f"volumerhs!: {name} has dims {arr.dims}, expected {dims}")
    st = L.lib.rk_volumerhs_f32(rhs.ptr, Q.ptr, vgeo.ptr, float(gravity), D.ptr, nelem, stream_ptr())
    L.check(st, "rk_volumerhs_f32")
    return rhs


def plan_volumerhs(rhs: ROCArray, Q: ROCArray, vgeo: ROCArray, gravity, D: ROCArray, nelem: int):
    """Callable that repeats ``volumerhs!`` on fixed arrays with no per-call host work beyond the
    foreign call (the benchmark loop of perf/volumerhs.jl:199-202)."""
    args = (rhs.ptr, Q.ptr, vgeo.ptr, float(gravity), D.ptr, int(nelem))
    fn = L.lib.rk_volumerhs_f32

    def launch():
        L.check(fn(*args, stream_ptr()), "rk_volumerhs_f32")
    return launch
