"""Host mirror of ``Base.accumulate!/accumulate/cumsum/cumprod(::AnyROCArray)``
(src/kernels/accumulate.jl:1-8): defaults and eltype rule on the host, one call through the C ABI.
"""
from __future__ import annotations

import numpy as np

from . import _lib as L
from .array import ROCArray, note_waiting_call, stream_ptr, workspace
from .mapreduce import _scalar_buffer


_SCAN_OP = {"add": L.RK_OP_ADD, "mul": L.RK_OP_MUL, "max": L.RK_OP_MAX, "min": L.RK_OP_MIN,
            "and": L.RK_OP_AND, "or": L.RK_OP_OR, "xor": L.RK_OP_XOR}          # & | xor: integer element types and Bool
_BITWISE = ("and", "or", "xor")


def accumulate_eltype(op: str, dtype) -> np.dtype:
    """``promote_op(op, T, typeof(init))`` with the reference's default ``init = zero(eltype(A))``
    (accumulate.jl:1,4): the eltype is preserved (Int32 stays Int32 and wraps); Bool counts in Int64, and stays Bool
    under the bitwise operators (``&``, ``|``, ``xor`` of Bools are Bools)."""
    dt = np.dtype(dtype)
    return np.dtype(np.int64) if dt == np.bool_ and op not in _BITWISE else dt


def accumulate_(op: str, B: ROCArray, A: ROCArray, dims=None, init=None, inclusive: bool = True) -> ROCArray:
    """``accumulate!(op, B, A; dims, init)``; ``B`` may be ``A`` itself.  Returns ``B``."""
    if op not in _SCAN_OP or (op in _BITWISE and np.dtype(B.dtype).kind not in "iub"):
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"scan operator {op!r} over {B.dtype}")
    if B.dims != A.dims:
        raise L.DimensionMismatch(L.RK_ERR_DIMENSION, f"accumulate!: {B.dims} vs {A.dims}")
    if dims is None:
        if A.ndim != 1:
            raise ValueError("accumulate without dims needs a vector (Base semantics)")
        dims = 1
    if dims < 1:
        raise ValueError("dims must be >= 1")
    if len(A) == 0:
        return B
    _launch_accumulate(op, B, A, dims, init, inclusive)()
    return B


# 1- and 2-byte element types (Int8, UInt8, Int16, UInt16, Float16) are scanned by the same kernels as the rest: the
# library reads them narrow, scans in the next wider type -- sums and products wrap modulo 2^32 and the store keeps the
# low bits, which is the narrow type's own wrap-around; Float16 in Float32 with one rounding at the store
# (AcceleratedKernels rounds after every step; the contract is a tolerance either way) -- and stores them narrow.


def _launch_accumulate(op, B, A, dims, init, inclusive):
    from .views import ROCView
    if isinstance(A, ROCView) or isinstance(B, ROCView):
        # wrapper arrays laid out alike (accumulate!(+, transpose(B), transpose(A))): the dims are renumbered in the ABI
        from .mapreduce import _dense_strides
        astr = tuple(A.strides) if isinstance(A, ROCView) else _dense_strides(A.dims)
        bstr = tuple(B.strides) if isinstance(B, ROCView) else _dense_strides(B.dims)
        aptr = A.sptr if isinstance(A, ROCView) else A.ptr
        bptr = B.sptr if isinstance(B, ROCView) else B.ptr
        ws, ws_bytes = workspace(16 << 20)
        sargs = (_SCAN_OP[op], A.code, B.code, aptr, bptr, A.ndim, L.shape_array(A.dims), L.shape_array(astr), L.shape_array(bstr), int(dims),
                 1 if inclusive else 0, _scalar_buffer(init, B.dtype), ws, ws_bytes)

        def launch_strided():
            note_waiting_call()
            L.check(L.lib.rk_accumulate_strided(*sargs, stream_ptr()), "rk_accumulate_strided")
        return launch_strided
    bytes_needed = L.lib.rk_workspace_bytes(L.RK_KIND_ACCUMULATE, B.code, A.ndim, L.shape_array(A.dims),
                                            (1 << (dims - 1)) if dims <= A.ndim else 0)
    ws, ws_bytes = workspace(bytes_needed)
    ibuf = _scalar_buffer(init, B.dtype)
    args = (_SCAN_OP[op], A.code, B.code, A.ptr, B.ptr, A.ndim, L.shape_array(A.dims), int(dims), 1 if inclusive else 0,
            ibuf, ws, ws_bytes)
    fn = L.lib.rk_accumulate

    def launch():
        note_waiting_call()
        L.check(fn(*args, stream_ptr()), "rk_accumulate")
    return launch


def plan_accumulate(op: str, B: ROCArray, A: ROCArray, dims=None, init=None, inclusive: bool = True):
    """Validate once, return a callable that repeats ``accumulate!(op, B, A; dims, init)`` with no
    per-call host work beyond the foreign call."""
    if op not in _SCAN_OP or B.dims != A.dims or len(A) == 0:
        raise ValueError("plan_accumulate: unsupported operator, mismatched dims or empty input")
    if dims is None:
        dims = 1
    return _launch_accumulate(op, B, A, dims, init, inclusive)


def accumulate(op: str, A: ROCArray, dims=None, init=None, inclusive: bool = True) -> ROCArray:
    """``accumulate(op, A; dims, init)`` -> new ROCArray of eltype ``accumulate_eltype``."""
    B = ROCArray(dims=A.dims, dtype=accumulate_eltype(op, A.dtype))
    return accumulate_(op, B, A, dims=dims, init=init, inclusive=inclusive)


def cumsum(A: ROCArray, dims=None) -> ROCArray:
    """``cumsum(::AnyROCArray; dims)`` (accumulate.jl:7).  Eltype-preserving: Int32 wraps."""
    return accumulate("add", A, dims=dims)


def cumprod(A: ROCArray, dims=None) -> ROCArray:
    return accumulate("mul", A, dims=dims)
