"""Strided wrappers over a ROCArray: ``view(A, ranges...)``, ``transpose(A)``, ``PermutedDimsArray(A, perm)``.

In the reference these are ``SubArray`` / ``Transpose`` / ``PermutedDimsArray`` wrappers that broadcast handles through
``ROCArrayStyle`` (src/broadcast.jl:7-10: "any ROCArray or wrapper").  Here a wrapper is a (pointer, dims, element strides)
triple; it can be an operand or the destination of a broadcast (``rk_broadcast_strided``), and ``copy`` makes it dense.
Reductions, scans and the other dense kernels take dense arrays only: their ``ptr`` is what those ops read, and a view has none."""
from __future__ import annotations

import numpy as np

from . import _lib as L
from .array import ROCArray, dtype_code


class ROCView:
    __slots__ = ("parent", "offset", "dims", "strides", "dtype")

    def __init__(self, parent: ROCArray, offset: int, dims, strides):
        self.parent = parent                       # keeps the storage alive
        self.offset = int(offset)                  # elements from parent's first element
        self.dims = tuple(int(d) for d in dims)
        self.strides = tuple(int(s) for s in strides)
        self.dtype = parent.dtype

    @property
    def ndim(self) -> int:
        return len(self.dims)

    def __len__(self) -> int:
        return int(np.prod(self.dims, dtype=np.int64))

    @property
    def code(self) -> int:
        return dtype_code(self.dtype)

    @property
    def sptr(self) -> int:
        """Address of the view's first element (what the strided broadcast entry points take)."""
        return self.parent.ptr + self.offset * self.dtype.itemsize

    @property
    def ptr(self):
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "this operation needs a dense array: copy(view) first")

    def __repr__(self):
        return f"ROCView{{{self.dtype}}}{self.dims} strides={self.strides}"


def _as_view(A) -> ROCView:
    if isinstance(A, ROCView):
        return A
    strides, s = [], 1
    for n in A.dims:
        strides.append(s)
        s *= n
    return ROCView(A, 0, A.dims, strides)


def view(A, *index) -> ROCView:
    """``view(A, I...)`` with 1-based indices: an ``int`` fixes (and drops) a dimension, ``None`` is ``:``, a tuple
    ``(first, last)`` is ``first:last`` and ``(first, step, last)`` is ``first:step:last`` (step may be negative)."""
    v = _as_view(A)
    if len(index) != v.ndim:
        raise IndexError(f"view of a {v.ndim}-d array needs {v.ndim} indices")
    offset, dims, strides = v.offset, [], []
    for n, s, ix in zip(v.dims, v.strides, index):
        if ix is None:
            dims.append(n); strides.append(s)
        elif isinstance(ix, (int, np.integer)):
            if not 1 <= ix <= n:
                raise IndexError(f"BoundsError: index {ix} of extent {n}")
            offset += (int(ix) - 1) * s
        else:
            first, step, last = (ix[0], 1, ix[1]) if len(ix) == 2 else ix
            count = max((last - first) // step + 1, 0) if step != 0 else 0
            if count > 0 and not (1 <= first <= n and 1 <= first + (count - 1) * step <= n):
                raise IndexError(f"BoundsError: range {first}:{step}:{last} of extent {n}")
            offset += (first - 1) * s if count > 0 else 0
            dims.append(count); strides.append(s * step)
    return ROCView(v.parent, offset, dims, strides)


def PermutedDimsArray(A, perm) -> ROCView:
    """Lazy ``PermutedDimsArray(A, perm)`` (1-based perm): ``size(P, k) == size(A, perm[k])``."""
    v = _as_view(A)
    perm = tuple(int(p) for p in perm)
    if sorted(perm) != list(range(1, v.ndim + 1)):
        raise ValueError(f"no valid permutation of dimensions: {perm}")
    return ROCView(v.parent, v.offset, [v.dims[p - 1] for p in perm], [v.strides[p - 1] for p in perm])


def transpose(A) -> ROCView:
    """Lazy ``transpose(A)`` of a matrix, or of a vector as a 1 x n row (real element types: no conjugation)."""
    v = _as_view(A)
    if v.ndim == 1:
        return ROCView(v.parent, v.offset, (1, v.dims[0]), (0, v.strides[0]))
    if v.ndim != 2:
        raise ValueError("transpose needs a vector or a matrix")
    return PermutedDimsArray(v, (2, 1))


def copy(v: ROCView) -> ROCArray:
    """Dense copy of a wrapper (``copy(view)`` / ``Array`` of it go through the broadcast kernel)."""
    from .broadcast import lazy, materialize_
    return materialize_(ROCArray(dims=v.dims, dtype=v.dtype), lazy(v))
