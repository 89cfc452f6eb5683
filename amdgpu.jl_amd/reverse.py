"""Host mirror of ``Base.reverse`` / ``Base.reverse!`` on ROCArrays (src/kernels/reverse.jl:1-57): the
argument checks and the vector / N-d split live here, the data movement is ``rk_reverse``."""
from __future__ import annotations

import numpy as np

from . import _lib as L
from .array import ROCArray, similar, stream_ptr


def _mask(x: ROCArray, dims) -> int:
    if dims is None:                                       # dims=:  (reverse.jl:35,50)
        dims = range(1, x.ndim + 1)
    elif isinstance(dims, (int, np.integer)):
        dims = (int(dims),)
    try:
        dims = tuple(int(d) for d in dims)
    except TypeError:
        raise ValueError(f"Dimension `{dims}` is not an iterable.") from None       # reverse.jl:37-38
    if not all(1 <= d <= x.ndim for d in dims):
        raise ValueError(f"Dimension `{dims}` is not 1 <= dims <= {x.ndim}")         # reverse.jl:39-40
    m = 0
    for d in dims:
        m |= 1 << (d - 1)
    return m


def _call(x: ROCArray, y: ROCArray, mask: int):
    L.check(L.lib.rk_reverse(x.ptr, y.ptr, x.dtype.itemsize, x.ndim, L.shape_array(x.dims), mask, stream_ptr()), "rk_reverse")


def _range(x: ROCArray, start, stop):
    if x.ndim != 1:
        raise ValueError("reverse(x, start, stop) needs a vector")
    n = x.dims[0]
    stop = n if stop is None else int(stop)
    start = int(start)
    if not (1 <= start and stop <= n):
        raise IndexError(f"reverse range {start}:{stop} out of bounds for length {n}")
    return start, stop, n


def reverse(x: ROCArray, start=None, stop=None, *, dims=None) -> ROCArray:
    """``reverse(x)``, ``reverse(x, start, stop)`` for vectors (reverse.jl:5-18), ``reverse(x; dims)`` for
    arrays (reverse.jl:34-47).  Returns a new array."""
    y = similar(x)
    if len(x) == 0:
        return y
    if start is not None:
        start, stop, n = _range(x, start, stop)
        if start > 1:                                      # reverse.jl:13
            _call(x.view_range(1, start - 1), y.view_range(1, start - 1), 0)
        if stop < n:                                       # reverse.jl:14
            _call(x.view_range(stop + 1, n), y.view_range(stop + 1, n), 0)
        if stop >= start:
            _call(x.view_range(start, stop), y.view_range(start, stop), 1)
        return y
    _call(x, y, _mask(x, dims))                            # all flipped extents 1 -> a plain copy (reverse.jl:42)
    return y


def reverse_(x: ROCArray, start=None, stop=None, *, dims=None) -> ROCArray:
    """``reverse!(x)``, ``reverse!(x, start, stop)`` (reverse.jl:20-28), ``reverse!(x; dims)`` (:49-57)."""
    if len(x) == 0:
        return x
    if start is not None:
        start, stop, _ = _range(x, start, stop)
        if stop > start:
            v = x.view_range(start, stop)
            _call(v, v, 1)
        return x
    _call(x, x, _mask(x, dims))
    return x
