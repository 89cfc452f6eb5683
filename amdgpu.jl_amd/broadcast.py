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

import builtins

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
_COMPARE = {"<": L.RK_BC_LT, "<=": L.RK_BC_LE, ">": L.RK_BC_GT, ">=": L.RK_BC_GE, "==": L.RK_BC_EQ, "!=": L.RK_BC_NE}
_LOGIC = {"&": L.RK_BC_AND, "|": L.RK_BC_OR}
_PREDICATE = {"!": L.RK_BC_NOT, "isodd": L.RK_BC_ISODD, "iseven": L.RK_BC_ISEVEN, "isnan": L.RK_BC_ISNAN}
_MATH = ("sqrt", "exp", "log", "sin", "cos", "tanh", "inv")


class Broadcasted:
    """Lazy broadcast node: ``f`` applied to ``args`` (leaves: ROCArray or scalar)."""

    __slots__ = ("f", "args")
    # NumPy scalars must hand `np.float32(0.5) * lazy(x)` to __rmul__ untouched; without this NumPy
    # would treat the node as an object array and pass a Python float (Float64) instead of 0.5f0
    __array_ufunc__ = None

    def __init__(self, f, args):
        self.f = f
        self.args = tuple(args)

    def __bool__(self):
        # `if x > 0:` inside a traced closure would otherwise take the same branch for every element, silently
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "truth value of a lazy broadcast: control flow on element values "
                                 "cannot be traced (ifelse can)")

    # arithmetic builds the tree (Julia's dot operators)
    def __add__(self, o): return Broadcasted("+", (self, _leaf(o)))
    def __radd__(self, o): return Broadcasted("+", (_leaf(o), self))
    def __sub__(self, o): return Broadcasted("-", (self, _leaf(o)))
    def __rsub__(self, o): return Broadcasted("-", (_leaf(o), self))
    def __mul__(self, o): return Broadcasted("*", (self, _leaf(o)))
    def __rmul__(self, o): return Broadcasted("*", (_leaf(o), self))
    def __truediv__(self, o): return Broadcasted("/", (self, _leaf(o)))
    def __rtruediv__(self, o): return Broadcasted("/", (_leaf(o), self))
    def __pow__(self, o):
        # a literal 2 is Base.literal_pow(^, x, Val(2)) = x * x in Julia, not a call of pow
        if type(o) is int and o == 2:
            return Broadcasted("abs2", (self,))
        return Broadcasted("^", (self, _leaf(o)))
    def __neg__(self): return Broadcasted("neg", (self,))
    # comparisons and logic (.<  .==  .&  .!): Bool-valued nodes
    def __lt__(self, o): return Broadcasted("<", (self, _leaf(o)))
    def __le__(self, o): return Broadcasted("<=", (self, _leaf(o)))
    def __gt__(self, o): return Broadcasted(">", (self, _leaf(o)))
    def __ge__(self, o): return Broadcasted(">=", (self, _leaf(o)))
    def __eq__(self, o): return Broadcasted("==", (self, _leaf(o)))
    def __ne__(self, o): return Broadcasted("!=", (self, _leaf(o)))
    __hash__ = object.__hash__
    def __and__(self, o): return Broadcasted("&", (self, _leaf(o)))
    def __rand__(self, o): return Broadcasted("&", (_leaf(o), self))
    def __or__(self, o): return Broadcasted("|", (self, _leaf(o)))
    def __ror__(self, o): return Broadcasted("|", (_leaf(o), self))
    def __invert__(self): return Broadcasted("!", (self,))


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
    if f == "ifelse":
        return ifelse(*args)
    if f not in _BINARY and f not in _UNARY and f not in _COMPARE and f not in _LOGIC and f not in _PREDICATE:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"broadcast function {f!r}")
    return Broadcasted(f, tuple(_leaf(a) for a in args))


def _unary(name):
    def fn(x):
        return Broadcasted(name, (_leaf(x),))
    fn.__name__ = name
    return fn


exp, log, sin, cos, tanh, sqrt, abs_, abs2, inv = (_unary(n) for n in
                                                    ("exp", "log", "sin", "cos", "tanh", "sqrt", "abs", "abs2", "inv"))


isodd, iseven, isnan, not_ = (_unary(n) for n in ("isodd", "iseven", "isnan", "!"))


def ifelse(c, a, b): return Broadcasted("ifelse", (_leaf(c), _leaf(a), _leaf(b)))
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


class MapVar:
    """Stands for the element in ``mapreduce(f, op, A)``: ``f(lazy(MapVar(eltype)))`` traces f into a tree."""
    __slots__ = ("dtype",)

    def __init__(self, dtype):
        self.dtype = np.dtype(dtype)


def _leaf_dtype(o) -> np.dtype:
    return o.dtype if isinstance(o, _ARRAYS + (MapVar,)) else _scalar_dtype(o)


def promote_type(a, b) -> np.dtype:
    """Julia's ``promote_type`` on the element types in use here: a float beats any integer and the wider float
    wins; Bool yields to integers; the wider integer wins, the unsigned one at equal width."""
    a, b = np.dtype(a), np.dtype(b)
    if a == b:
        return a
    if a.kind == "f" or b.kind == "f":
        return max((d for d in (a, b) if d.kind == "f"), key=lambda d: d.itemsize)
    if a.kind == "b":
        return b
    if b.kind == "b":
        return a
    if a.itemsize != b.itemsize:
        return a if a.itemsize > b.itemsize else b
    return a if a.kind == "u" else b


def _infer(bc: Broadcasted, types: dict) -> np.dtype:
    """Julia's result eltype of every node of the tree (``Broadcast.combine_eltypes``), by node identity."""
    if bc.f is None:
        t = _leaf_dtype(bc.args[0])
    else:
        ats = [_infer(a, types) for a in bc.args]
        t = ats[0]
        for u in ats[1:]:
            t = promote_type(t, u)
        if bc.f in _COMPARE or bc.f in _LOGIC or bc.f in _PREDICATE:
            if bc.f in ("isodd", "iseven") and ats[0].kind == "f":
                raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"{bc.f} of floating-point values")
            t = np.dtype(np.bool_)
        elif bc.f == "ifelse":
            t = promote_type(ats[1], ats[2])
        elif bc.f in ("/", "^") or bc.f in _MATH:
            if t.kind != "f":
                t = np.dtype(np.float64)               # Int / Int and sqrt(Int) are Float64
        elif bc.f in ("+", "-", "*", "muladd", "neg") and t.kind == "b":
            t = np.dtype(np.int64)                     # true + true isa Int
    if t.kind not in "fiub":
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"broadcast over eltype {t}")
    types[id(bc)] = t
    return t


_ORDER_SENSITIVE = set(_COMPARE) | set(_LOGIC) | {"!", "max", "min"}


def _emit(bc: Broadcasted, operands: list, tokens: list, types: dict, int_program: bool):
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
        _emit(a, operands, tokens, types, int_program)
        # integer programs compute in Int64: where the order or the zero-ness of a 32-bit intermediate matters,
        # bring it back to the value Julia holds (Int32 arithmetic wraps)
        if int_program and bc.f in _ORDER_SENSITIVE and a.f is not None:
            _wrap(types[id(a)], tokens)
    if bc.f == "muladd":
        tokens.append(L.RK_BC_FMA)
    elif bc.f == "ifelse":
        tokens.append(L.RK_BC_IFELSE)
    else:
        for table in (_BINARY, _UNARY, _COMPARE, _LOGIC, _PREDICATE):
            if bc.f in table:
                tokens.append(table[bc.f])
                break
    # Julia computes Float16 arithmetic in Float32 and rounds every result: so does the program
    if types[id(bc)] == np.float16 and (bc.f in ("+", "-", "*", "/", "^", "muladd", "abs2") or bc.f in _MATH):
        tokens.append(L.RK_BC_ROUND_F16)


_WRAP_TOKEN = {np.dtype(np.int32): L.RK_BC_WRAP_I32, np.dtype(np.uint32): L.RK_BC_WRAP_U32,
               np.dtype(np.int8): L.RK_BC_WRAP_I8, np.dtype(np.uint8): L.RK_BC_WRAP_U8,
               np.dtype(np.int16): L.RK_BC_WRAP_I16, np.dtype(np.uint16): L.RK_BC_WRAP_U16}


def _wrap(t: np.dtype, tokens: list):
    tok = _WRAP_TOKEN.get(np.dtype(t))
    if tok is not None:
        tokens.append(tok)


def _compile_tree(tree: Broadcasted, operands: list):
    """Type the tree and flatten it after the operands already listed; returns (tokens, compute type, result eltype).
    Floating-point programs compute in the promoted float type.  All-integer programs compute in Int64 and keep
    Julia's result eltype (Int32 .+ Int32 is an Int32 that wraps); with ``/`` or a math function Julia's result is
    a Float64, and so is the compute type here."""
    types: dict = {}
    eltype = _infer(tree, types)
    kinds = list(types.values())
    floats = [t for t in kinds if t.kind == "f"]
    if floats:
        compute = max(floats, key=lambda d: d.itemsize)
        if compute == np.float16:
            compute = np.dtype(np.float32)             # with RK_BC_ROUND_F16 after every Float16-typed operation
    else:
        compute = np.dtype(np.int64)
    tokens: list = []
    _emit(tree, operands, tokens, types, not floats)
    if not floats:
        # an order-sensitive token over UInt64 values cannot be computed in Int64
        def visit(n):
            if n.f in _ORDER_SENSITIVE and builtins.any(types[id(a)] == np.uint64 for a in n.args):
                raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"{n.f} of UInt64 values")
            if n.f is not None:
                for a in n.args:
                    visit(a)
        visit(tree)
    return tokens, compute, eltype, types


def _compile(bc: Broadcasted):
    """Flatten ``bc``; returns (operands, tokens, compute type, shape, result eltype)."""
    operands: list = []
    tokens, compute, eltype, _ = _compile_tree(_leaf(bc), operands)
    if len(tokens) > L.RK_MAX_PROGRAM:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "broadcast expression too long")
    shapes = [o.dims for o in operands if isinstance(o, _ARRAYS)]
    return operands, tokens, compute, broadcast_shape(*shapes), eltype


def compile_map(f, dtype):
    """Trace the unary closure ``f`` of ``mapreduce(f, op, A)`` on a symbolic element: returns
    (tokens, constants, Julia's eltype of f(x), compute type).  Token 0 is the element, tokens 1.. the constants;
    a closure that captures an array, needs more than RK_MAP_MAX_CONSTS constants, RK_MAP_MAX_TOKENS tokens or a
    deeper value stack than the kernels keep in registers is unsupported."""
    var = MapVar(dtype)
    tree = _leaf(f(lazy(var)))
    operands: list = [var]
    tokens, compute, eltype, types = _compile_tree(tree, operands)
    consts = operands[1:]
    if builtins.any(isinstance(c, _ARRAYS + (MapVar,)) for c in consts):
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "mapreduce closure over an array")
    if compute.kind != "f" and tree.f is not None:
        _wrap(eltype, tokens)                          # the reduction sees the Int32 Julia would hand it
    if len(tokens) > L.RK_MAP_MAX_TOKENS or len(consts) > L.RK_MAP_MAX_CONSTS:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "mapreduce closure too long")
    return tokens, consts, eltype, compute


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


def _extent(a):
    """(first byte, one past the last byte, identity of the layout) of the memory an array or wrapper addresses."""
    size = a.dtype.itemsize
    if isinstance(a, ROCView):
        lo = hi = a.sptr
        for n, st in zip(a.dims, a.strides):
            if n == 0:
                return a.sptr, a.sptr, None
            span = (n - 1) * st * size
            lo, hi = (lo + span, hi) if span < 0 else (lo, hi + span)
        return lo, hi + size, (a.sptr, a.dims, a.strides)
    dense, st = [], 1
    for n in a.dims:
        dense.append(st)
        st *= n
    return a.ptr, a.ptr + len(a) * size, (a.ptr, a.dims, tuple(dense))


def _unalias(dest, operands):
    """``Broadcast.broadcast_unalias``: an operand that may share memory with the destination without being the very
    same elements in the same places (``x .= x .+ 1`` is fine; ``@view(A[1:4, :]) .= @view(A[2:5, :])`` is not) is
    copied first, so the kernel never reads an element another lane has already overwritten."""
    from .views import copy as copy_view
    dlo, dhi, dident = _extent(dest)
    out = []
    for o in operands:
        if isinstance(o, _ARRAYS) and len(o) > 0 and dhi > dlo:
            lo, hi, ident = _extent(o)
            if lo < dhi and dlo < hi and ident != dident:
                o = copy_view(o) if isinstance(o, ROCView) else o.copy()
        out.append(o)
    return out


def _launch_broadcast(dest, operands, tokens, compute, repeatable=False):
    fresh = _unalias(dest, operands)
    if repeatable and builtins.any(a is not b for a, b in zip(fresh, operands)):
        # a plan would keep reading the copy made now
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "a prepared broadcast whose operand aliases the destination")
    operands = fresh
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
    return _launch_broadcast(dest, operands, tokens, compute, repeatable=True)


def materialize(bc) -> ROCArray:
    """``Broadcast.materialize(bc)``: allocates the result (``similar(bc, T, dims)``, broadcast.jl:26-30)."""
    operands, tokens, compute, shape, eltype = _compile(bc)
    dest = ROCArray(dims=shape, dtype=eltype)
    return materialize_(dest, bc)


def fill_(dest: ROCArray, value) -> ROCArray:
    """``fill!(dest, value)`` / ``dest .= value`` (benchmarked as ``gpu_mat .= 0f0``, perf/array.jl:67)."""
    return materialize_(dest, lazy(value))
