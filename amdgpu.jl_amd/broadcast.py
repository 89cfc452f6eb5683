"""Host mirror of fused broadcast on ROCArray (src/broadcast.jl:3-35).

Julia builds a lazy ``Broadcasted`` tree for ``z .= a .* x .+ y .* exp.(w)`` and hands it to
``copyto!(dest, bc)``.  Here the tree is built with :func:`lazy` leaves and Python operators, then
flattened to the postfix program of the C ABI and executed by ONE fused kernel::

    materialize_(z, a * lazy(x) + lazy(y) * exp(lazy(w)))     # z .= a .* x .+ y .* exp.(w)
    C = materialize(lazy(A) + lazy(r) * lazy(c))              # C = A .+ r .* c

Shape rule = Julia's: dims align from the first; an extent of 1 (or a missing trailing dim) is
extruded.  Scalars: NumPy scalars keep their type (``np.float32(0.5)`` is ``0.5f0``), Python floats
are Float64 and Python ints Int64, as in Julia.
"""
from __future__ import annotations

import numpy as np

from . import _lib as L
from .array import ROCArray, dtype_code, stream_ptr
from .views import ROCView

_ARRAYS = (ROCArray, ROCView)

_BINARY = {"+": L.RK_BC_ADD, "-": L.RK_BC_SUB, "*": L.RK_BC_MUL, "/": L.RK_BC_DIV, "max": L.RK_BC_MAX,
           "min": L.RK_BC_MIN, "^": L.RK_BC_POW}
_UNARY = {"neg": L.RK_BC_NEG, "abs": L.RK_BC_ABS, "abs2": L.RK_BC_ABS2, "sqrt": L.RK_BC_SQRT, "exp": L.RK_BC_EXP,
          "log": L.RK_BC_LOG, "sin": L.RK_BC_SIN, "cos": L.RK_BC_COS, "tanh": L.RK_BC_TANH, "inv": L.RK_BC_INV,
          "identity": L.RK_BC_IDENTITY}


class Broadcasted:
    """Lazy broadcast node: ``f`` applied to ``args`` (leaves: ROCArray or scalar)."""

    __slots__ = ("f", "args")
    # NumPy scalars must hand `np.float32(0.5) * lazy(x)` to __rmul__ untouched; without this NumPy
    # would treat the node as an object array and pass a Python float (Float64) instead of 0.5f0
    __array_ufunc__ = None

    def __init__(self, f, args):
        self.f = f
        self.args = tuple(args)

    # arithmetic builds the tree (Julia's dot operators)
    def __add__(self, o): return Broadcasted("+", (self, _leaf(o)))
    def __radd__(self, o): return Broadcasted("+", (_leaf(o), self))
    def __sub__(self, o): return Broadcasted("-", (self, _leaf(o)))
    def __rsub__(self, o): return Broadcasted("-", (_leaf(o), self))
    def __mul__(self, o): return Broadcasted("*", (self, _leaf(o)))
    def __rmul__(self, o): return Broadcasted("*", (_leaf(o), self))
    def __truediv__(self, o): return Broadcasted("/", (self, _leaf(o)))
    def __rtruediv__(self, o): return Broadcasted("/", (_leaf(o), self))
    def __pow__(self, o): return Broadcasted("^", (self, _leaf(o)))
    def __neg__(self): return Broadcasted("neg", (self,))


def _leaf(x):
    if isinstance(x, Broadcasted):
        return x
    return Broadcasted(None, (x,))


def lazy(x) -> Broadcasted:
    """Wrap a ROCArray or scalar as a broadcast leaf."""
    return _leaf(x)


def broadcasted(f: str, *args) -> Broadcasted:
    """``Broadcast.broadcasted(f, args...)`` for an enumerated ``f``."""
    if f == "muladd":
        return Broadcasted("muladd", tuple(_leaf(a) for a in args))
    if f not in _BINARY and f not in _UNARY:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"broadcast function {f!r}")
    return Broadcasted(f, tuple(_leaf(a) for a in args))


def _unary(name):
    def fn(x):
        return Broadcasted(name, (_leaf(x),))
    fn.__name__ = name
    return fn


exp, log, sin, cos, tanh, sqrt, abs_, abs2, inv = (_unary(n) for n in
                                                    ("exp", "log", "sin", "cos", "tanh", "sqrt", "abs", "abs2", "inv"))


def max_(a, b): return Broadcasted("max", (_leaf(a), _leaf(b)))
def min_(a, b): return Broadcasted("min", (_leaf(a), _leaf(b)))
def muladd(a, b, c): return Broadcasted("muladd", (_leaf(a), _leaf(b), _leaf(c)))


def _scalar_dtype(v) -> np.dtype:
    if isinstance(v, (bool, np.bool_)):
        return np.dtype(np.bool_)
    if isinstance(v, np.generic):
        return v.dtype
    if isinstance(v, int):
        return np.dtype(np.int64)
    if isinstance(v, float):
        return np.dtype(np.float64)
    raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"broadcast operand of type {type(v).__name__}")


def broadcast_shape(*shapes):
    """``Broadcast.broadcast_shape``: align from the first dim; 1 extrudes; else DimensionMismatch."""
    nd = max((len(s) for s in shapes), default=0)
    out = []
    for d in range(nd):
        ext = 1
        for s in shapes:
            n = s[d] if d < len(s) else 1
            if n != 1:
                if ext != 1 and ext != n:
                    raise L.DimensionMismatch(L.RK_ERR_DIMENSION, f"arrays could not be broadcast to a common size: {shapes}")
                ext = n
        out.append(ext)
    return tuple(out)


def _flatten(bc: Broadcasted, operands: list, tokens: list):
    if bc.f is None:
        leaf = bc.args[0]
        for k, o in enumerate(operands):           # the same array object appears once
            if o is leaf:
                tokens.append(k)
                return
        if len(operands) >= L.RK_MAX_OPERANDS:
            raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "more than 8 broadcast operands")
        operands.append(leaf)
        tokens.append(len(operands) - 1)
        return
    for a in bc.args:
        _flatten(a, operands, tokens)
    if bc.f == "muladd":
        tokens.append(L.RK_BC_FMA)
    elif bc.f in _BINARY:
        tokens.append(_BINARY[bc.f])
    else:
        tokens.append(_UNARY[bc.f])


_INT_SAFE = None


def _int_safe_tokens():
    global _INT_SAFE
    if _INT_SAFE is None:
        _INT_SAFE = {L.RK_BC_ADD, L.RK_BC_SUB, L.RK_BC_MUL, L.RK_BC_MAX, L.RK_BC_MIN, L.RK_BC_FMA,
                     L.RK_BC_NEG, L.RK_BC_ABS, L.RK_BC_ABS2, L.RK_BC_IDENTITY}
    return _INT_SAFE


def _compile(bc: Broadcasted):
    """Flatten ``bc``; returns (operands, tokens, compute type, shape, result eltype).  Floating-point programs compute
    in the promoted float type.  All-integer programs of ``+ - * max min muladd - abs abs2`` compute in Int64 and keep
    Julia's result eltype (Int32 .+ Int32 is an Int32 that wraps); with ``/`` or a math function Julia's result is a
    Float64, and so is the compute type here."""
    operands, tokens = [], []
    _flatten(_leaf(bc), operands, tokens)
    if len(tokens) > L.RK_MAX_PROGRAM:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "broadcast expression too long")
    dts = [o.dtype if isinstance(o, _ARRAYS) else _scalar_dtype(o) for o in operands]
    eltype = np.result_type(*dts) if dts else np.dtype(np.float64)
    compute = eltype
    ops = [t for t in tokens if t >= L.RK_MAX_OPERANDS]
    if eltype.kind != "f":
        if eltype.kind not in "iub":
            raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"broadcast over eltype {eltype}")
        if all(t in _int_safe_tokens() for t in ops):
            if eltype == np.uint64 and any(t in (L.RK_BC_MAX, L.RK_BC_MIN) for t in ops):
                raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "max / min of UInt64 values")
            compute = np.dtype(np.int64)
            if eltype == np.bool_ and ops:             # true + true isa Int
                eltype = np.dtype(np.int64)
        else:
            compute = eltype = np.dtype(np.float64)
    if compute == np.float16:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "Float16 broadcast")
    shapes = [o.dims for o in operands if isinstance(o, _ARRAYS)]
    return operands, tokens, compute, broadcast_shape(*shapes), eltype


def _program(operands, tokens, compute, dest_ndim) -> L.RkProgram:
    p = L.RkProgram()
    p.compute = dtype_code(compute)
    p.n_operands = len(operands)
    for k, o in enumerate(operands):
        ro = p.operands[k]
        if isinstance(o, _ARRAYS):
            ro.ptr = o.sptr if isinstance(o, ROCView) else o.ptr
            ro.dtype = o.code
            dims = o.dims
            while len(dims) > dest_ndim and dims[-1] == 1:     # trailing singleton dims carry nothing
                dims = dims[:-1]
            ro.ndim = len(dims)
            for d, n in enumerate(dims):
                ro.shape[d] = n
            if isinstance(o, ROCView):                         # SubArray / Transpose / PermutedDimsArray operand
                ro.strided = 1
                for d in range(len(dims)):
                    ro.strides[d] = o.strides[d]
        else:
            dt = _scalar_dtype(o)
            ro.ptr = None
            ro.dtype = dtype_code(dt)
            ro.ndim = 0
            if dt.kind == "f":
                ro.scalar_f = float(o)
            else:
                ro.scalar_i = int(o)
    p.n_tokens = len(tokens)
    for i, t in enumerate(tokens):
        p.tokens[i] = t
    return p


def materialize_(dest: ROCArray, bc) -> ROCArray:
    """``Broadcast.materialize!(dest, bc)`` / ``copyto!(dest, bc)``: one fused kernel, returns dest."""
    operands, tokens, compute, shape, _ = _compile(bc)
    full = broadcast_shape(shape, dest.dims)
    while len(full) > dest.ndim and full[-1] == 1:
        full = full[:-1]
    if full != dest.dims:
        raise L.DimensionMismatch(L.RK_ERR_DIMENSION, f"destination {dest.dims} vs broadcast shape {shape}")
    if len(dest) == 0:
        return dest
    _launch_broadcast(dest, operands, tokens, compute)()
    return dest


def _launch_broadcast(dest, operands, tokens, compute):
    prog = _program(operands, tokens, compute, dest.ndim)
    keep = operands          # the program holds raw device pointers: keep the arrays alive with the plan
    if isinstance(dest, ROCView):                  # `@view(C[...]) .= bc`, `transpose(C) .= bc`
        args = (prog, dest.sptr, dest.code, dest.ndim, L.shape_array(dest.dims), L.shape_array(dest.strides))
        fn, name = L.lib.rk_broadcast_strided, "rk_broadcast_strided"
    else:
        args = (prog, dest.ptr, dest.code, dest.ndim, L.shape_array(dest.dims))
        fn, name = L.lib.rk_broadcast, "rk_broadcast"

    def launch(_keep=keep):
        L.check(fn(*args, stream_ptr()), name)
    return launch


def plan_materialize(dest: ROCArray, bc):
    """Flatten and validate ``dest .= bc`` once; the returned callable repeats it with no per-call host
    work beyond the foreign call (Julia specialises the same tree at compile time)."""
    operands, tokens, compute, shape, _ = _compile(bc)
    full = broadcast_shape(shape, dest.dims)
    while len(full) > dest.ndim and full[-1] == 1:
        full = full[:-1]
    if full != dest.dims or len(dest) == 0:
        raise L.DimensionMismatch(L.RK_ERR_DIMENSION, f"destination {dest.dims} vs broadcast shape {shape}")
    return _launch_broadcast(dest, operands, tokens, compute)


def materialize(bc) -> ROCArray:
    """``Broadcast.materialize(bc)``: allocates the result (``similar(bc, T, dims)``, broadcast.jl:26-30)."""
    operands, tokens, compute, shape, eltype = _compile(bc)
    dest = ROCArray(dims=shape, dtype=eltype)
    return materialize_(dest, bc)


def fill_(dest: ROCArray, value) -> ROCArray:
    """``fill!(dest, value)`` / ``dest .= value`` (benchmarked as ``gpu_mat .= 0f0``, perf/array.jl:67)."""
    return materialize_(dest, lazy(value))
