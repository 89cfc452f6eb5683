"""Host mirror of ``permutedims`` / ``permutedims!`` on ROCArrays (Base semantics; the reference runs GPUArrays'
generic kernel for it, perf/array.jl:151-155): checks here, data movement in ``rk_permutedims``."""
from __future__ import annotations

import ctypes as C

from . import _lib as L
from .array import ROCArray, stream_ptr


def _check_perm(ndim: int, perm) -> tuple:
    perm = tuple(int(p) for p in perm)
    if len(perm) != ndim or sorted(perm) != list(range(1, ndim + 1)):
        raise ValueError(f"no valid permutation of dimensions: {perm} for {ndim} dims")     # Base's ArgumentError
    return perm


def permutedims_(dest: ROCArray, src: ROCArray, perm) -> ROCArray:
    """``permutedims!(dest, src, perm)``: ``size(dest, k) == size(src, perm[k])``; returns ``dest``."""
    perm = _check_perm(src.ndim, perm)
    want = tuple(src.dims[p - 1] for p in perm)
    if dest.dims != want or dest.dtype != src.dtype:
        raise L.DimensionMismatch(L.RK_ERR_DIMENSION, f"permutedims!: destination {dest.dims} vs {want}")
    if len(src) == 0:
        return dest
    parr = (C.c_int32 * max(len(perm), 1))(*perm)
    L.check(L.lib.rk_permutedims(src.ptr, dest.ptr, src.dtype.itemsize, src.ndim, L.shape_array(src.dims), parr, stream_ptr()),
            "rk_permutedims")
    return dest


def permutedims(src: ROCArray, perm=None) -> ROCArray:
    """``permutedims(src, perm)``; ``permutedims(m)`` of a matrix is its transpose copy, of a vector a 1 x n row."""
    if perm is None:
        if src.ndim == 1:
            return ROCArray(buf=src.copy().buf, dims=(1, src.dims[0]), dtype=src.dtype)
        if src.ndim != 2:
            raise ValueError("permutedims without perm needs a vector or a matrix")
        perm = (2, 1)
    perm = _check_perm(src.ndim, perm)
    dest = ROCArray(dims=tuple(src.dims[p - 1] for p in perm), dtype=src.dtype)
    return permutedims_(dest, src, perm)
