"""Host mirror of the reduction front end: Base.mapreduce / sum / maximum / findmax on ROCArray and
``GPUArrays.mapreducedim!`` (src/kernels/mapreduce.jl:86-173).

Everything here is argument plumbing that the Julia front end does before the kernel runs --
eltype and ``init`` selection (``Base.add_sum`` widens Int32 to Int64), the shape of ``R`` with
singleton reduced dims (mapreduce.jl:95-107), the scalar fetch for ``dims=:`` -- followed by one call
through the C ABI.  No arithmetic happens on the host.
"""
from __future__ import annotations

import builtins
import ctypes as C

import numpy as np

from . import _lib as L
from .array import ROCArray, dtype_code, stream_ptr, workspace

# f of mapreduce(f, op, A): enumerated, like the C ABI
identity, abs2, abs_ = "identity", "abs2", "abs"
# op: "add_sum"/"mul_prod" are what sum/prod use (they widen small integers), "add"/"mul" keep the eltype
add_sum, mul_prod, add, mul, max_, min_ = "add_sum", "mul_prod", "add", "mul", "max", "min"

_MAP = {"identity": L.RK_MAP_IDENTITY, "abs2": L.RK_MAP_ABS2, "abs": L.RK_MAP_ABS}
_OP = {"add_sum": L.RK_OP_ADD, "add": L.RK_OP_ADD, "mul_prod": L.RK_OP_MUL, "mul": L.RK_OP_MUL,
       "max": L.RK_OP_MAX, "min": L.RK_OP_MIN}


def reduce_eltype(op: str, dtype) -> np.dtype:
    """``promote_op(op, T, T)`` as GPUArrays' ``_mapreduce`` infers it: add_sum / mul_prod widen
    Int8..Int32 and Bool to Int64 (UInt8..UInt32 to UInt64); ``+``/``*``/``max``/``min`` keep T."""
    dt = np.dtype(dtype)
    if op in ("add_sum", "mul_prod"):
        if dt == np.bool_ or dt.type in (np.int8, np.int16, np.int32):
            return np.dtype(np.int64)
        if dt.type in (np.uint8, np.uint16, np.uint32):
            return np.dtype(np.uint64)
        return dt
    if op in ("add", "mul") and dt == np.bool_:
        return np.dtype(np.int64)
    if op not in _OP:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"reduction operator {op!r}")
    return dt


def _dims_mask(dims, ndim: int) -> int:
    if dims is None:
        return (1 << ndim) - 1
    if isinstance(dims, (int, np.integer)):
        dims = (int(dims),)
    mask = 0
    for d in dims:
        if d < 1:
            raise ValueError("dims must be >= 1")
        if d <= ndim:
            mask |= 1 << (d - 1)
    return mask


def _reduced_dims(dims_in, mask):
    return tuple(1 if (mask >> d) & 1 else n for d, n in enumerate(dims_in))


def _dense_strides(dims):
    out, s = [], 1
    for n in dims:
        out.append(s)
        s *= n
    return tuple(out)


def _scalar_buffer(value, dtype: np.dtype):
    """Host scalar of ``dtype`` as a ctypes buffer (the ABI reads it during the call)."""
    if value is None:
        return None
    return C.create_string_buffer(np.array(value, dtype=dtype).tobytes(), dtype.itemsize)


def _map_program(f, dtype):
    """A closure for f -> (rk_map_program, Julia's eltype of f(x)); traced by calling it on a symbolic element."""
    from .broadcast import compile_map
    tokens, consts, eltype, compute = compile_map(f, dtype)
    if builtins.any(t in (L.RK_BC_POW, L.RK_BC_SIN, L.RK_BC_COS, L.RK_BC_TANH) for t in tokens):
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "pow / sin / cos / tanh inside a reduction kernel")
    dt = np.dtype(dtype)
    if (compute.kind == "f") != (dt.kind == "f") or (compute.kind == "f" and compute != dt):
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"mapreduce closure computing in {compute} over {dt} elements "
                                                       "(a Python float is a Float64: use np.float32 constants)")
    p = L.RkMapProgram()
    p.n_tokens = len(tokens)
    for i, t in enumerate(tokens):
        p.tokens[i] = t
    p.n_consts = len(consts)
    for k, c in enumerate(consts):
        if compute.kind == "f":
            p.const_f[k] = float(c)
        else:
            p.const_i[k] = int(c)
    return p, eltype


def mapreducedim_(f, op: str, R: ROCArray, A: ROCArray, init=None) -> ROCArray:
    """``GPUArrays.mapreducedim!(f, op, R, A; init)``: reduces A into R over every dimension in which
    R has extent 1 and A does not; returns the R object it was given (mapreduce.jl:93,172;
    test/core/rocarray_base.jl:263-267).  With ``init=None`` the neutral element of ``op`` is used.
    ``f`` is one of the enumerated maps or a closure of the element (``lambda x: x + 1``)."""
    if not callable(f) and f not in _MAP:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"map {f!r}")
    if op not in _OP:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, f"reduction operator {op!r}")
    # Base.check_reducedims (mapreduce.jl:90)
    rdims = R.dims + (1,) * (A.ndim - R.ndim)          # pad with singleton dims (mapreduce.jl:95-98)
    if len(rdims) != A.ndim:
        raise L.DimensionMismatch(L.RK_ERR_DIMENSION, "mapreducedim!: R has more dimensions than A")
    mask = 0
    for d, (r, a) in enumerate(zip(rdims, A.dims)):
        if r == a:
            continue
        if r != 1:
            raise L.DimensionMismatch(L.RK_ERR_DIMENSION, f"mapreducedim!: cannot reduce {A.dims} into {R.dims}")
        mask |= 1 << d
    if len(A) == 0:
        return R                                        # mapreduce.jl:91
    _launch_mapreducedim(f, op, R, A, init, mask)()
    return R


def _launch_mapreducedim(f, op, R, A, init, mask):
    """Zero-argument callable that enqueues the reduction on the current stream."""
    ws, ws_bytes = workspace()
    ibuf = _scalar_buffer(init, R.dtype)
    from .views import ROCView
    if isinstance(R, ROCView) or isinstance(A, ROCView):
        # wrapper arrays (transpose, PermutedDimsArray): rk_mapreduce_strided renumbers the dims; closures for f and
        # views with gaps are not native here
        if callable(f):
            raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "a closure for f over a wrapper array: copy(view) first")
        rdims = tuple(R.dims) + (1,) * (A.ndim - R.ndim)
        rstr = (tuple(R.strides) if isinstance(R, ROCView) else _dense_strides(R.dims)) + (0,) * (A.ndim - R.ndim)
        astr = tuple(A.strides) if isinstance(A, ROCView) else _dense_strides(A.dims)
        rstr = tuple(s if n > 1 else 0 for s, n in zip(rstr, rdims))
        aptr = A.sptr if isinstance(A, ROCView) else A.ptr
        rptr = R.sptr if isinstance(R, ROCView) else R.ptr
        args = (_MAP[f], _OP[op], A.code, R.code, aptr, A.ndim, L.shape_array(A.dims), L.shape_array(astr), mask, rptr,
                L.shape_array(rstr), ibuf, ws, ws_bytes)
        fn, name = L.lib.rk_mapreduce_strided, "rk_mapreduce_strided"

        def launch_strided():
            L.check(fn(*args, stream_ptr()), name)
        return launch_strided
    if callable(f):
        prog, _ = _map_program(f, A.dtype)
        args = (prog, _OP[op], A.code, R.code, A.ptr, A.ndim, L.shape_array(A.dims), mask, R.ptr, ibuf, ws, ws_bytes)
        fn, name = L.lib.rk_mapreduce_program, "rk_mapreduce_program"
    else:
        args = (_MAP[f], _OP[op], A.code, R.code, A.ptr, A.ndim, L.shape_array(A.dims), mask, R.ptr, ibuf, ws, ws_bytes)
        fn, name = L.lib.rk_mapreduce, "rk_mapreduce"

    def launch():
        L.check(fn(*args, stream_ptr()), name)
    return launch


def plan_mapreducedim(f: str, op: str, R: ROCArray, A: ROCArray, init=None):
    """Validate once, return a callable that repeats ``mapreducedim!(f, op, R, A; init)`` with no
    per-call host work beyond the foreign call (what a compiled ``ccall`` site costs in Julia)."""
    rdims = R.dims + (1,) * (A.ndim - R.ndim)
    mask = 0
    for d, (r, a) in enumerate(zip(rdims, A.dims)):
        if r != a:
            if r != 1:
                raise L.DimensionMismatch(L.RK_ERR_DIMENSION, f"mapreducedim!: cannot reduce {A.dims} into {R.dims}")
            mask |= 1 << d
    return _launch_mapreducedim(f, op, R, A, init, mask)


def mapreduce(f, op: str, A: ROCArray, dims=None, init=None):
    """``mapreduce(f, op, A; dims, init)``.  ``dims=None`` is Julia's ``:`` and returns a host scalar
    (a blocking 4/8-byte read, like ``@allowscalar R[]`` in GPUArrays); otherwise a ROCArray whose
    reduced dims have extent 1.  ``f``: "identity" / "abs2" / "abs", or a closure of the element built from
    arithmetic, comparisons and this package's functions (``lambda x: x + 1``, ``lambda x: isodd(x)``): it is
    traced into a program that the reduction kernels evaluate on the loaded values (one pass over A); the result
    eltype is ``promote_op(op, T, T)`` with T the eltype of ``f(x)``, as GPUArrays infers it."""
    mask = _dims_mask(dims, A.ndim)
    if callable(f):
        try:
            _, mapped = _map_program(f, A.dtype)
        except L.UnsupportedError:
            # a closure the reduction kernels do not interpret (too long, pow or trigonometry, another array, a result
            # in another float type): map first -- one fused broadcast kernel -- then reduce the mapped array
            from .broadcast import lazy, materialize
            return mapreduce(identity, op, materialize(f(lazy(A))), dims=dims, init=init)
        if mapped == np.bool_ and op in ("max", "min"):
            return _reduce_predicate(f, op, A, dims, mask)
        out_dt = reduce_eltype(op, mapped)
    else:
        out_dt = reduce_eltype(op, A.dtype)
    if len(A) == 0:
        if op in ("max", "min"):
            raise ValueError("reducing over an empty collection is not allowed")
        neutral = init if init is not None else (0 if _OP[op] == L.RK_OP_ADD else 1)
        if dims is None:
            return out_dt.type(neutral)
        R = ROCArray(np.full(_reduced_dims(A.dims, mask), neutral, dtype=out_dt))
        return R
    rshape = (1,) * A.ndim if dims is None else _reduced_dims(A.dims, mask)
    R = ROCArray(dims=rshape, dtype=out_dt)
    mapreducedim_(f, op, R, A, init=init)
    if dims is None:
        return R.item()
    return R


def _reduce_predicate(pred, op, A, dims, mask):
    """``any(pred, A; dims)`` / ``all(pred, A; dims)``: | and & of Bools are max and min of 0 / 1, accumulated in A's
    own element type (Int64 for Bool arrays) and turned into Bools at the end."""
    from .broadcast import lazy, materialize
    acc_dt = A.dtype if A.dtype in (np.float32, np.float64, np.int32, np.int64) else np.dtype(np.int64)
    if len(A) == 0:
        neutral = op == "min"
        return neutral if dims is None else ROCArray(np.full(_reduced_dims(A.dims, mask), neutral, dtype=np.bool_))
    rshape = (1,) * A.ndim if dims is None else _reduced_dims(A.dims, mask)
    R = ROCArray(dims=rshape, dtype=acc_dt)
    mapreducedim_(pred, op, R, A)
    if dims is None:
        return bool(R.item() != 0)
    return materialize(lazy(R) != acc_dt.type(0))


def _split(args, name):
    """(f, A) from Julia's two call forms ``name(A)`` and ``name(f, A)``."""
    if len(args) == 1:
        return None, args[0]
    if len(args) == 2 and callable(args[0]):
        return args
    raise TypeError(f"{name}(A) or {name}(f, A)")


def sum(*args, dims=None, f=identity):          # noqa: A001 - mirrors Base.sum
    """``sum(A; dims)`` / ``sum(f, A; dims)``."""
    g, A = _split(args, "sum")
    return mapreduce(g if g is not None else f, add_sum, A, dims=dims)


def prod(*args, dims=None):
    g, A = _split(args, "prod")
    return mapreduce(g if g is not None else identity, mul_prod, A, dims=dims)


def maximum(*args, dims=None):
    g, A = _split(args, "maximum")
    return mapreduce(g if g is not None else identity, max_, A, dims=dims)


def minimum(*args, dims=None):
    g, A = _split(args, "minimum")
    return mapreduce(g if g is not None else identity, min_, A, dims=dims)


def _predicate_or_bools(pred, A, name):
    """(pred, A) when the reduction kernels interpret ``pred``; (None, pred.(A)) -- the Bools materialized by one
    broadcast kernel -- when they do not."""
    try:
        _, mapped = _map_program(pred, A.dtype)
    except L.UnsupportedError:
        from .broadcast import lazy, materialize
        pred, A = None, materialize(pred(lazy(A)))
        mapped = A.dtype
    if mapped != np.bool_:
        raise TypeError(f"{name}: non-boolean ({mapped}) used in boolean context")     # Julia's TypeError
    return pred, A


def count(*args, dims=None):
    """``count(::ROCArray{Bool}; dims)`` == sum of the Bool array in Int64; ``count(pred, A; dims)`` sums the
    predicate's Bools in the same single pass over A."""
    pred, A = _split(args, "count")
    if pred is not None:
        pred, A = _predicate_or_bools(pred, A, "count")
    if pred is not None:
        return mapreduce(pred, add_sum, A, dims=dims)
    if A.dtype != np.bool_:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "count needs a Bool array")
    return mapreduce(identity, add_sum, A, dims=dims)


def any(*args, dims=None):                             # noqa: A001 - mirrors Base.any
    """``any(::ROCArray{Bool}; dims)``: ``|`` over Bools is ``max`` over their bytes.  ``any(pred, A; dims)``."""
    pred, A = _split(args, "any")
    if pred is not None:
        pred, A = _predicate_or_bools(pred, A, "any")
    if pred is not None:
        return mapreduce(pred, max_, A, dims=dims)
    if A.dtype != np.bool_:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "any needs a Bool array or a predicate")
    if len(A) == 0:
        return False if dims is None else ROCArray(np.zeros(_reduced_dims(A.dims, _dims_mask(dims, A.ndim)), dtype=np.bool_))
    r = mapreduce(identity, max_, A, dims=dims)
    return bool(r) if dims is None else r


def all(*args, dims=None):                             # noqa: A001 - mirrors Base.all
    """``all(::ROCArray{Bool}; dims)``: ``&`` over Bools is ``min`` over their bytes.  ``all(pred, A; dims)``."""
    pred, A = _split(args, "all")
    if pred is not None:
        pred, A = _predicate_or_bools(pred, A, "all")
    if pred is not None:
        return mapreduce(pred, min_, A, dims=dims)
    if A.dtype != np.bool_:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "all needs a Bool array or a predicate")
    if len(A) == 0:
        return True if dims is None else ROCArray(np.ones(_reduced_dims(A.dims, _dims_mask(dims, A.ndim)), dtype=np.bool_))
    r = mapreduce(identity, min_, A, dims=dims)
    return bool(r) if dims is None else r


def findfirst(*args):
    """``findfirst(::ROCArray{Bool})``: index of the first true entry in column-major order (an Int for
    vectors, a CartesianIndex tuple otherwise) or ``None``: the argmax of the bytes, ties to the smallest index.
    ``findfirst(pred, A)`` searches ``pred.(A)`` (benchmarked in perf/array.jl:44-47)."""
    pred, A = _split(args, "findfirst")
    if pred is not None:
        from .broadcast import lazy, materialize
        A = materialize(pred(lazy(A)))
        if A.dtype != np.bool_:
            raise TypeError(f"findfirst: non-boolean ({A.dtype}) used in boolean context")
    if A.dtype != np.bool_:
        raise L.UnsupportedError(L.RK_ERR_UNSUPPORTED, "findfirst needs a Bool array or a predicate")
    if len(A) == 0:
        return None
    v, i = _findminmax(A, True, None)
    return i if v else None


def _findminmax(A, want_max: bool, dims):
    if len(A) == 0:
        raise ValueError("reducing over an empty collection is not allowed")
    mask = _dims_mask(dims, A.ndim)
    rshape = (1,) * A.ndim if dims is None else _reduced_dims(A.dims, mask)
    vals = ROCArray(dims=rshape, dtype=A.dtype)
    # Array{CartesianIndex{N}}: N Int64 per element; kept as an Int64 array with a leading dim N
    idx = ROCArray(dims=(A.ndim,) + rshape, dtype=np.int64)
    ws, ws_bytes = workspace()
    from .views import ROCView
    if isinstance(A, ROCView):
        # wrapper arrays (transpose, PermutedDimsArray): the index comes back in the wrapper's coordinates; orders of
        # dims for which the first of equal winners or the output layout would differ raise UnsupportedError
        st = L.lib.rk_findminmax_strided(1 if want_max else 0, A.code, A.sptr, A.ndim, L.shape_array(A.dims),
                                         L.shape_array(tuple(A.strides)), mask, vals.ptr, idx.ptr, ws, ws_bytes, stream_ptr())
        L.check(st, "rk_findminmax_strided")
    else:
        st = L.lib.rk_findminmax(1 if want_max else 0, A.code, A.ptr, A.ndim, L.shape_array(A.dims), mask,
                                 vals.ptr, idx.ptr, ws, ws_bytes, stream_ptr())
        L.check(st, "rk_findminmax")
    if dims is None:
        c = tuple(int(v) for v in idx.to_host().reshape(-1))
        return vals.item(), (c[0] if A.ndim == 1 else c)
    return vals, idx


def findmax(A, dims=None):
    """``findmax(A; dims)``: (values, indices).  With ``dims``: ``values`` is a ROCArray with reduced
    dims of extent 1 and ``indices`` an Int64 ROCArray of dims ``(ndims(A), size(values)...)`` whose
    column ``[:, I]`` is the CartesianIndex of the winner.  Without: host scalar and index tuple
    (an Int for vectors)."""
    return _findminmax(A, True, dims)


def findmin(A, dims=None):
    return _findminmax(A, False, dims)


def argmax(A: ROCArray, dims=None):
    """``argmax(A; dims)`` = the index half of ``findmax`` (the kernel skips the value output)."""
    return _findminmax(A, True, dims)[1]


def argmin(A: ROCArray, dims=None):
    return _findminmax(A, False, dims)[1]


def extrema(*args, dims=None):
    """``extrema(A; dims)`` / ``extrema(f, A; dims)``: (minimum, maximum) -- host scalars, or two ROCArrays with
    ``dims`` (Julia returns one array of tuples; the pair of arrays holds the same values)."""
    return minimum(*args, dims=dims), maximum(*args, dims=dims)


def plan_findmax(A: ROCArray, vals: ROCArray, idx: ROCArray, dims, want_max: bool = True):
    """Callable that repeats ``findmax(A; dims)`` into preallocated outputs."""
    mask = _dims_mask(dims, A.ndim)
    ws, ws_bytes = workspace()
    args = (1 if want_max else 0, A.code, A.ptr, A.ndim, L.shape_array(A.dims), mask, vals.ptr, idx.ptr, ws, ws_bytes)
    fn = L.lib.rk_findminmax

    def launch():
        L.check(fn(*args, stream_ptr()), "rk_findminmax")
    return launch
