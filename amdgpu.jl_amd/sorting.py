"""Host mirror of ``Base.sort!`` / ``sort`` / ``sortperm!`` / ``sortperm`` on ROC vectors
(src/kernels/sorting.jl:1-3).  The default order and ``rev`` go to the native radix sort.  The two other forms the
reference's own test runs (test/hip_rocarray/sorting.jl:20-26) are native too: ``lt=!isless`` (here ``lt=not_isless``)
is the descending order, and ``by=k -> 2k`` -- any ``by`` the broadcast machinery can evaluate -- sorts the keys
``by.(x)`` with ``sortperm`` and gathers: map, radix sort of (key, index) pairs, gather.  Any other ``lt`` raises
``UnsupportedError`` (the Julia shim keeps the stock path for it)."""
from __future__ import annotations

import numpy as np
import torch

from . import _lib as L
from .array import ROCArray, device, note_sort, stream_ptr


def isless(a, b):          # the default ``lt``; only its identity matters here
    raise TypeError("isless is a marker for sort's lt keyword, not a host function")


def not_isless(a, b):      # Julia's ``!isless``: as ``lt`` it orders descending (equal keys in no particular order)
    raise TypeError("not_isless is a marker for sort's lt keyword, not a host function")


def _check(x: ROCArray, lt, by) -> bool:
    """Validates the keywords; returns True when ``lt`` reverses the order."""
    if lt is not None and lt is not isless and lt is not not_isless:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "sort with a custom lt (other than isless / !isless)")
    if x.ndim != 1:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "sort of an N-d array (dims=) is not on the GPU path of the reference either")
    return lt is not_isless


def _keys(x: ROCArray, by) -> ROCArray:
    """``by.(x)`` through the fused broadcast (raises UnsupportedError for a ``by`` it cannot express)."""
    from .broadcast import lazy, materialize
    return materialize(by(lazy(x)))


def _gather(x: ROCArray, perm: ROCArray) -> ROCArray:
    y = ROCArray(dims=x.dims, dtype=x.dtype)
    n = len(x)
    if n > 0:
        L.check(L.lib.rk_gather_slices(x.ptr, perm.ptr, y.ptr, x.dtype.itemsize, 1, n, n, stream_ptr()), "rk_gather_slices")
    return y


def _tmp(code: int, n: int, perm: bool) -> torch.Tensor:
    nbytes = int(L.lib.rk_sort_tmp_bytes(code, n, 1 if perm else 0))
    t = torch.empty(nbytes, dtype=torch.uint8, device=device())
    assert t.data_ptr() % 256 == 0
    return t


def _release(tmp: torch.Tensor, n: int) -> None:
    """Sorts of up to 2^20 keys resolve their digit offsets by look-back, with bounded waits: their temporary is kept
    until its give-up record has been read (``array.check_waits``, at the next ``Array(x)``).  Larger sorts count
    before every pass and wait for nobody: their temporary goes back to the allocator at once."""
    if n <= (1 << 20):
        note_sort(tmp)
    else:
        tmp.record_stream(torch.cuda.current_stream())


def sort_(x: ROCArray, *, rev: bool = False, lt=None, by=None) -> ROCArray:
    """``sort!(x; rev, lt, by)``: in place, returns ``x``."""
    rev = bool(rev) != _check(x, lt, by)
    n = len(x)
    if by is not None and n > 1:
        y = _gather(x, sortperm(_keys(x, by), rev=rev))
        x.buf[x.offset:x.offset + n * x.dtype.itemsize].copy_(y.buf[:n * x.dtype.itemsize])
        return x
    if n > 1:
        tmp = _tmp(x.code, n, False)
        L.check(L.lib.rk_sort(x.code, x.ptr, n, 1 if rev else 0, tmp.data_ptr(), tmp.numel(), stream_ptr()), "rk_sort")
        _release(tmp, n)
    return x


def sort(x: ROCArray, *, rev: bool = False, lt=None, by=None) -> ROCArray:
    """``sort(x; rev, lt, by)``: sorted copy."""
    rev = bool(rev) != _check(x, lt, by)
    if by is not None:
        return _gather(x, sortperm(_keys(x, by), rev=rev)) if len(x) > 1 else x.copy()
    return sort_(x.copy(), rev=rev)


def sortperm_(ix: ROCArray, x: ROCArray, *, rev: bool = False, lt=None, by=None) -> ROCArray:
    """``sortperm!(ix, x; rev, lt, by)``: ``ix`` (Int64, length of ``x``) receives the 1-based stable permutation."""
    rev = bool(rev) != _check(x, lt, by)
    if by is not None:
        x = _keys(x, by)
    if ix.dtype != np.int64 or ix.dims != x.dims:
        raise L.DimensionMismatch(L.RK_ERR_DIMENSION, "sortperm!: ix must be an Int64 vector of the length of x")
    n = len(x)
    if n > 0:
        tmp = _tmp(x.code, n, True)
        L.check(L.lib.rk_sortperm(x.code, x.ptr, ix.ptr, n, 1 if rev else 0, tmp.data_ptr(), tmp.numel(), stream_ptr()), "rk_sortperm")
        _release(tmp, n)
    return ix


def sortperm(x: ROCArray, *, rev: bool = False, lt=None, by=None) -> ROCArray:
    """``sortperm(x; rev, lt, by)`` (sorting.jl:3)."""
    return sortperm_(ROCArray(dims=x.dims, dtype=np.int64), x, rev=rev, lt=lt, by=by)
