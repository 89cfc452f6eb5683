"""Host mirror of ``Base.findall(::AnyROCArray{Bool})`` (src/kernels/indexing.jl:8-36): a cumsum over
the flattened Bool array (the scan of this path), a scalar fetch of the count, then the scatter kernel."""
from __future__ import annotations

import numpy as np

from . import _lib as L
from .accumulate import accumulate
from .array import ROCArray, stream_ptr


def findall(bools: ROCArray) -> ROCArray:
    """1-based indices of the true entries, in column-major order: an Int64 vector for vectors, an
    Int64 ``(N, count)`` array of CartesianIndex columns for N-d arrays (``keytype(bools)``)."""
    if bools.dtype != np.bool_:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "findall needs a Bool array")
    n = len(bools)
    nd = bools.ndim
    if n == 0:
        return ROCArray(dims=(0,) if nd == 1 else (nd, 0), dtype=np.int64)
    flat = bools.reshape(n)
    indices = accumulate("add", flat)                       # indexing.jl:10
    count = int(indices.view_range(n, n).item())            # indexing.jl:12 (@allowscalar indices[end])
    ys = ROCArray(dims=(count,) if nd == 1 else (nd, count), dtype=np.int64)
    if count > 0:
        st = L.lib.rk_findall_scatter(bools.ptr, indices.ptr, ys.ptr, nd, L.shape_array(bools.dims), stream_ptr())
        L.check(st, "rk_findall_scatter")
    return ys

