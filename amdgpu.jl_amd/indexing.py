"""Host mirror of ``Base.findall(::AnyROCArray{Bool})`` (src/kernels/indexing.jl:8-36).

``findall`` is the one-pass form: count the true entries (a U8 -> Int64 reduction), fetch the count,
allocate, then one stream-compaction pass (``rk_findall``).  ``findall_two_pass`` keeps the reference's
own structure -- Int64 cumsum of the flattened mask, scalar fetch of its last entry, scatter kernel -- on
the native scan and ``rk_findall_scatter``."""
from __future__ import annotations

import numpy as np

from . import _lib as L
from .accumulate import accumulate
from .array import ROCArray, note_waiting_call, stream_ptr, workspace
from .mapreduce import count


def _empty(nd: int) -> ROCArray:
    return ROCArray(dims=(0,) if nd == 1 else (nd, 0), dtype=np.int64)


def findall(*args) -> ROCArray:
    """1-based indices of the true entries, in column-major order: an Int64 vector for vectors, an
    Int64 ``(N, count)`` array of CartesianIndex columns for N-d arrays (``keytype(bools)``).
    ``findall(pred, A)`` is ``findall(pred.(A))`` (benchmarked in perf/array.jl:39-42)."""
    if len(args) == 2 and callable(args[0]):
        from .broadcast import lazy, materialize
        bools = materialize(args[0](lazy(args[1])))
    else:
        (bools,) = args
    if bools.dtype != np.bool_:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "findall needs a Bool array")
    n, nd = len(bools), bools.ndim
    if n == 0:
        return _empty(nd)
    total = int(count(bools))                                # indexing.jl:12 (the scalar fetch)
    ys = ROCArray(dims=(total,) if nd == 1 else (nd, total), dtype=np.int64)
    if total > 0:
        shape = L.shape_array(bools.dims)
        ws, ws_bytes = workspace(L.lib.rk_workspace_bytes(L.RK_KIND_FINDALL, L.RK_U8, nd, shape, 0))
        note_waiting_call()
        L.check(L.lib.rk_findall(bools.ptr, nd, shape, ys.ptr, None, ws, ws_bytes, stream_ptr()), "rk_findall")
    return ys


def findall_two_pass(bools: ROCArray) -> ROCArray:
    """The reference's sequence of kernels: cumsum (indexing.jl:10), count fetch (:12), scatter (:16-31)."""
    if bools.dtype != np.bool_:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "findall needs a Bool array")
    n, nd = len(bools), bools.ndim
    if n == 0:
        return _empty(nd)
    indices = accumulate("add", bools.reshape(n))
    total = int(indices.view_range(n, n).item())
    ys = ROCArray(dims=(total,) if nd == 1 else (nd, total), dtype=np.int64)
    if total > 0:
        st = L.lib.rk_findall_scatter(bools.ptr, indices.ptr, ys.ptr, nd, L.shape_array(bools.dims), stream_ptr())
        L.check(st, "rk_findall_scatter")
    return ys


def getindex_mask(x: ROCArray, mask: ROCArray) -> ROCArray:
    """``x[mask]`` for a mask of x's shape, or ``x[:, ..., :, mask]`` for a Bool vector along the last dim
    (test/hip_rocarray/indexing.jl:5-18): ``Base.to_index`` turns the mask into ``findall(mask)``
    (indexing.jl:1), then the selected slices are gathered."""
    if mask.dtype != np.bool_:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "logical indexing needs a Bool mask")
    if mask.dims == x.dims:
        inner, nsrc, lead = 1, len(x), ()
        idx = findall(mask.reshape(len(mask)))
    elif mask.ndim == 1 and x.ndim >= 1 and mask.dims[0] == x.dims[-1]:
        lead = x.dims[:-1]
        inner, nsrc = int(np.prod(lead, dtype=np.int64)), x.dims[-1]
        idx = findall(mask)
    else:
        raise IndexError(f"BoundsError: mask {mask.dims} against array {x.dims}")       # Base.checkbounds
    n = len(idx)
    y = ROCArray(dims=lead + (n,), dtype=x.dtype)
    if n > 0 and inner > 0:
        L.check(L.lib.rk_gather_slices(x.ptr, idx.ptr, y.ptr, x.dtype.itemsize, inner, n, nsrc, stream_ptr()), "rk_gather_slices")
    return y
