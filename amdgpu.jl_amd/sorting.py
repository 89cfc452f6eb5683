"""Host mirror of ``Base.sort!`` / ``sort`` / ``sortperm!`` / ``sortperm`` on ROC vectors
(src/kernels/sorting.jl:1-3).  The default order and ``rev`` go to the native radix sort; ``lt`` and ``by``
closures have no native form and raise ``UnsupportedError`` (the Julia shim keeps the stock path for them)."""
from __future__ import annotations

import numpy as np
import torch

from . import _lib as L
from .array import ROCArray, device, note_sort, stream_ptr


def _check(x: ROCArray, lt, by):
    if lt is not None or by is not None:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "sort with a custom lt / by")
    if x.ndim != 1:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "sort of an N-d array (dims=) is not on the GPU path of the reference either")


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
    """``sort!(x; rev)``: in place, returns ``x``."""
    _check(x, lt, by)
    n = len(x)
    if n > 1:
        tmp = _tmp(x.code, n, False)
        L.check(L.lib.rk_sort(x.code, x.ptr, n, 1 if rev else 0, tmp.data_ptr(), tmp.numel(), stream_ptr()), "rk_sort")
        _release(tmp, n)
    return x


def sort(x: ROCArray, *, rev: bool = False, lt=None, by=None) -> ROCArray:
    """``sort(x; rev)``: sorted copy."""
    _check(x, lt, by)
    return sort_(x.copy(), rev=rev)


def sortperm_(ix: ROCArray, x: ROCArray, *, rev: bool = False, lt=None, by=None) -> ROCArray:
    """``sortperm!(ix, x; rev)``: ``ix`` (Int64, length of ``x``) receives the 1-based stable permutation."""
    _check(x, lt, by)
    if ix.dtype != np.int64 or ix.dims != x.dims:
        raise L.DimensionMismatch(L.RK_ERR_DIMENSION, "sortperm!: ix must be an Int64 vector of the length of x")
    n = len(x)
    if n > 0:
        tmp = _tmp(x.code, n, True)
        L.check(L.lib.rk_sortperm(x.code, x.ptr, ix.ptr, n, 1 if rev else 0, tmp.data_ptr(), tmp.numel(), stream_ptr()), "rk_sortperm")
        _release(tmp, n)
    return ix


def sortperm(x: ROCArray, *, rev: bool = False, lt=None, by=None) -> ROCArray:
    """``sortperm(x; rev)`` (sorting.jl:3)."""
    _check(x, lt, by)
    return sortperm_(ROCArray(dims=x.dims, dtype=np.int64), x, rev=rev)
