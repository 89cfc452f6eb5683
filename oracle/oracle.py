"""CPU oracle for the ROCArray array-kernel path -- TEST INFRASTRUCTURE ONLY.

This module restates, in NumPy (Float64 / exact integers), what the reference's
array-kernel layer computes.  It is the checker that the HIP kernels are compared
against; it is never the thing measured or shipped.  Only tests/, the smoke test and
the CPU-baseline leg of the benchmark may import it.

The reference (AMDGPU.jl, Julia) cannot run in this environment: there is no Julia
runtime, and the arithmetic of three of the four op families lives in packages that are
not vendored in the reference tree (GPUArrays.jl, AcceleratedKernels.jl;
Project.toml:54,62 give compat ranges only).  Every op on this path is *defined* by the
reference's own tests as "equal to Julia Base on Array" (test/runtests.jl:77-82,
`testf` compares ROCArray against Array), so each function below restates Julia Base
semantics and cites the reference call site whose contract it follows.

Conventions
-----------
* Arrays are NumPy arrays carrying Julia's *logical* shape ``(d1, ..., dn)``; memory
  order is irrelevant here (the device layout is column-major, see the host package).
* ``dims`` are 1-based like Julia's; indices returned are 1-based.
* Float results are produced in Float64 (the comparison tolerance lives in the tests);
  integer results are exact in the output type Julia would pick.

How each function is pinned (see tests/test_oracle.py):

=====================  ==========================================================
function               pinned by
=====================  ==========================================================
reduce_eltype          Base rule table + docs/src/usage/arrays.md:85-89 doctests
mapreduce / sum        doctests sum(1:100)=5050, mapreduce(x->x^2,+,1:4)=30
                       (docs/src/usage/arrays.md:85-89); sum(ones)=n
                       (test/hip_rocarray/multi_gpu.jl:45,48); closed forms;
                       brute-force Python loops on tiny inputs
maximum / findmax      brute-force sequential Base._rf_findmax loop on tiny inputs
                       with planted ties, NaNs and signed zeros
accumulate / cumsum    doctest cumsum([1,2,3,4])=[1,3,6,10] (arrays.md:91-96);
                       sequential loops for the sizes and dims cases of
                       test/core/rocarray_base.jl:194-225; Int32 wraparound by
                       modular closed form
broadcast              per-element scalar loops for the extrusion cases of
                       test/core/rocarray_broadcast.jl:19-20
findall                np.nonzero brute force vs test/hip_rocarray/indexing.jl:5-18
volumerhs              two independent restatements (literal loop transcription
                       vs tensor-contraction form) + the constant-state invariant
                       + linearity in D + a hand-computed single-node case
=====================  ==========================================================

Parity unpinned (no check in the reference tree can pin them, stated here as required):
* GPUArrays' own findmax corner cases where they may deviate from Base
  (``isless(-0.0, 0.0)``, NaN payloads).  This oracle follows **Base**.
* the exact Float32 bit patterns the reference GPU kernels produce (tree order).
  The contract is a tolerance against Float64, not bit patterns.
"""
from __future__ import annotations

import numpy as np

# ---------------------------------------------------------------------------
# eltype rules  (front end of src/kernels/mapreduce.jl:86; GPUArrays `_mapreduce`
# infers ET = promote_op(op, T, T); Base.add_sum widens small integers)
# ---------------------------------------------------------------------------

_SMALL_SIGNED = (np.int8, np.int16, np.int32)
_SMALL_UNSIGNED = (np.uint8, np.uint16, np.uint32)


def reduce_eltype(op: str, dtype) -> np.dtype:
    """Output eltype of ``mapreduce(identity, op, A)`` for Julia eltype ``dtype``.

    ``add_sum`` / ``mul_prod`` (what ``sum`` / ``prod`` use) widen Int8..Int32 to
    Int64, UInt8..UInt32 to UInt64 and Bool to Int64; plain ``+``/``*``/``max``/``min``
    keep the eltype.  Floats are never widened.
    """
    dt = np.dtype(dtype)
    if op in ("add_sum", "mul_prod"):
        if dt == np.bool_:
            return np.dtype(np.int64)
        if dt.type in _SMALL_SIGNED:
            return np.dtype(np.int64)
        if dt.type in _SMALL_UNSIGNED:
            return np.dtype(np.uint64)
        return dt
    if op in ("add", "mul"):
        if dt == np.bool_:
            return np.dtype(np.int64)  # true + true isa Int
        return dt
    if op in ("max", "min"):
        return dt
    raise ValueError(f"unknown op {op!r}")


def accumulate_eltype(op: str, dtype) -> np.dtype:
    """Output eltype of ``accumulate(op, A)`` on a ROCArray.

    src/kernels/accumulate.jl:1-8 passes ``init = zero(eltype(A))`` to AcceleratedKernels,
    which allocates ``promote_op(op, T, typeof(init))``: the eltype is preserved
    (Int32 stays Int32 and wraps), only Bool promotes to Int64.
    """
    dt = np.dtype(dtype)
    if dt == np.bool_ and op not in ("and", "or", "xor"):     # &, |, xor of Bools are Bools
        return np.dtype(np.int64)
    return dt


# ---------------------------------------------------------------------------
# mapreduce  (src/kernels/mapreduce.jl:86-173)
# ---------------------------------------------------------------------------

def _normalize_dims(dims, ndim):
    """Julia ``dims`` (Colon == None, Int or tuple, 1-based) -> sorted 0-based axes.

    Dimensions beyond ``ndim`` are legal in Julia and reduce nothing.
    """
    if dims is None:
        return tuple(range(ndim))
    if isinstance(dims, (int, np.integer)):
        dims = (int(dims),)
    out = []
    for d in dims:
        if d < 1:
            raise ValueError("dims must be >= 1")
        if d <= ndim:
            out.append(d - 1)
    return tuple(sorted(set(out)))


def _apply_map(f: str, a: np.ndarray) -> np.ndarray:
    if f == "identity":
        return a
    if f == "abs2":
        return a * a
    if f == "abs":
        return np.abs(a)
    raise ValueError(f"unknown map {f!r}")


def _wide(a: np.ndarray, out_dtype: np.dtype) -> np.ndarray:
    """Promote to the precision the oracle computes in."""
    if out_dtype.kind == "f":
        return a.astype(np.float64)
    if out_dtype.kind in "iub":                  # (b: Bool under the bitwise scan operators)
        return a.astype(out_dtype)
    raise ValueError(out_dtype)


def julia_max(a, b):
    """Base.max on floats: NaN-propagating, max(-0.0, 0.0) == 0.0."""
    if np.isnan(a) or np.isnan(b):
        return np.nan
    if a == b:  # picks +0.0 over -0.0
        return b if np.signbit(a) else a
    return a if a > b else b


def julia_min(a, b):
    if np.isnan(a) or np.isnan(b):
        return np.nan
    if a == b:
        return a if np.signbit(a) else b
    return a if a < b else b


def mapreduce(f: str, op: str, A: np.ndarray, dims=None, init=None) -> np.ndarray:
    """``mapreduce(f, op, A; dims, init)`` with Base semantics.

    Follows the shape contract of ``GPUArrays.mapreducedim!``
    (src/kernels/mapreduce.jl:95-107): the result keeps every reduced dimension as a
    singleton.  With ``dims=None`` (Julia's ``:``) the result is a 0-d array holding
    the scalar (the front end fetches ``R[]``).  An empty ``A`` returns ``R`` filled
    with the neutral element / ``init`` (mapreduce.jl:91).

    Float inputs are accumulated in Float64, integers exactly in the output eltype
    (two's-complement wraparound like Julia).
    """
    A = np.asarray(A)
    axes = _normalize_dims(dims, A.ndim)
    out_dt = reduce_eltype(op, A.dtype)
    if A.dtype.kind in "iu":
        # f runs on the element, in the element type: abs2(x::Int16) is an Int16 and wraps; add_sum widens afterwards
        with np.errstate(over="ignore"):
            a = _wide(_apply_map(f, A).astype(A.dtype), out_dt)
    else:
        a = _apply_map(f, _wide(A, out_dt))
    base = {"add_sum": "add", "mul_prod": "mul"}.get(op, op)
    with np.errstate(over="ignore"):
        if base == "add":
            r = a.sum(axis=axes, keepdims=True, dtype=a.dtype)
            if init is not None:
                r = r + a.dtype.type(init)
        elif base == "mul":
            r = a.prod(axis=axes, keepdims=True, dtype=a.dtype)
            if init is not None:
                r = r * a.dtype.type(init)
        elif base in ("max", "min"):
            if a.size == 0:
                raise ValueError("reducing over an empty collection is not allowed")
            if a.dtype.kind == "f":
                # np.max propagates NaN like Base.max, and IEEE max of +-0 may pick
                # either; fix the signed-zero case explicitly.
                r = (np.max if base == "max" else np.min)(a, axis=axes, keepdims=True)
                zero_hit = (r == 0)
                if np.any(zero_hit):
                    if base == "max":
                        has = np.any((a == 0) & ~np.signbit(a), axis=axes, keepdims=True)
                        r = np.where(zero_hit & has, 0.0, np.where(zero_hit, -0.0, r))
                    else:
                        has = np.any((a == 0) & np.signbit(a), axis=axes, keepdims=True)
                        r = np.where(zero_hit & has, -0.0, np.where(zero_hit, 0.0, r))
            else:
                r = (np.max if base == "max" else np.min)(a, axis=axes, keepdims=True)
            if init is not None:
                fn = np.maximum if base == "max" else np.minimum
                r = fn(r, a.dtype.type(init))
        else:
            raise ValueError(f"unknown op {op!r}")
    if dims is None:
        return r.reshape(())
    return r


def sum_(A, dims=None):
    """``sum(A; dims)`` == ``mapreduce(identity, Base.add_sum, A; dims)``."""
    return mapreduce("identity", "add_sum", A, dims=dims)


def maximum(A, dims=None):
    return mapreduce("identity", "max", A, dims=dims)


def minimum(A, dims=None):
    return mapreduce("identity", "min", A, dims=dims)


# ---------------------------------------------------------------------------
# findmax / findmin   (front end: GPUArrays findminmax -> mapreducedim! with a
# (value, CartesianIndex) tuple, src/kernels/mapreduce.jl:86; semantics: Base)
# ---------------------------------------------------------------------------

def _isless(a, b) -> bool:
    """Base.isless total order on floats: -0.0 < 0.0, NaN is greater than everything."""
    an, bn = np.isnan(a), np.isnan(b)
    if an or bn:
        return (not an) and bn
    if a == b:
        return bool(np.signbit(a)) and not bool(np.signbit(b))
    return bool(a < b)


def _order_score(A: np.ndarray, want_max: bool) -> np.ndarray:
    """Int64 score whose *largest* value marks the findmax (findmin) winner.

    Floats follow Base's total order: ``isless`` has -0.0 < 0.0 and NaN above
    everything, so for ``findmax`` NaN wins; ``findmin`` uses ``isgreater``, under
    which NaN wins as well (``findmin([1, NaN]) == (NaN, 2)``).
    """
    A = np.asarray(A)
    if A.dtype.kind == "f":
        if A.dtype == np.float16:
            A = A.astype(np.float32)                    # exact, and order-preserving
        if A.dtype == np.float32:
            bits = A.view(np.int32).astype(np.int64)
            mag = bits & np.int64(0x7FFFFFFF)
        elif A.dtype == np.float64:
            bits = A.view(np.int64)
            mag = bits & np.int64(0x7FFFFFFFFFFFFFFF)
        else:
            raise TypeError(A.dtype)
        key = np.where(bits < 0, -mag - 1, mag)         # monotone in isless order
        score = key if want_max else ~key
        return np.where(np.isnan(A), np.iinfo(np.int64).max, score)
    if A.dtype == np.uint64:
        key = (A ^ np.uint64(1 << 63)).view(np.int64)
    else:
        key = A.astype(np.int64)
    return key if want_max else ~key


def findminmax(A: np.ndarray, want_max: bool, dims=None):
    """``findmax(A; dims)`` / ``findmin(A; dims)`` with Base semantics.

    Returns ``(values, index)``.  With ``dims=None``: ``values`` is a scalar of A's
    eltype and ``index`` the 1-based CartesianIndex as a tuple (a plain int for
    vectors).  With ``dims``: ``values`` has A's shape with reduced dims singleton and
    ``index`` is an Int64 array of shape ``values.shape + (ndim,)`` holding 1-based
    Cartesian coordinates.  Ties resolve to the first index in column-major iteration
    order; the first NaN wins; +0.0 beats -0.0 for max (Base._rf_findmax / isless).
    """
    A = np.asarray(A)
    if A.size == 0:
        raise ValueError("reducing over an empty collection is not allowed")
    nd = A.ndim
    axes = _normalize_dims(dims, nd)
    kept = tuple(i for i in range(nd) if i not in axes)
    score = _order_score(A, want_max)
    lin = np.arange(A.size, dtype=np.int64).reshape(A.shape, order="F")
    kshape = tuple(A.shape[i] for i in kept)
    perm = kept + axes
    sc = np.transpose(score, perm).reshape(kshape + (-1,))
    ln = np.transpose(lin, perm).reshape(kshape + (-1,))
    # visit every reduced block in column-major order so that "first" is well defined
    order = np.argsort(ln, axis=-1, kind="stable")
    sc = np.take_along_axis(sc, order, axis=-1)
    ln = np.take_along_axis(ln, order, axis=-1)
    pos = np.argmax(sc, axis=-1)                         # first occurrence of the best
    win = np.take_along_axis(ln, pos[..., None], axis=-1)[..., 0]
    vals = A.reshape(-1, order="F")[win]
    coords = np.stack(np.unravel_index(win, A.shape, order="F"), axis=-1).astype(np.int64) + 1
    if dims is None:
        c = tuple(int(v) for v in coords.reshape(-1))
        return A.dtype.type(vals.reshape(())), (c[0] if nd == 1 else c)
    out_shape = tuple(1 if i in axes else A.shape[i] for i in range(nd))
    # kept axes are in increasing order, so a plain reshape restores the layout
    return vals.reshape(out_shape), coords.reshape(out_shape + (nd,))


def findmax(A, dims=None):
    return findminmax(A, True, dims)


def findmin(A, dims=None):
    return findminmax(A, False, dims)


# ---------------------------------------------------------------------------
# accumulate / cumsum / cumprod   (src/kernels/accumulate.jl:1-8)
# ---------------------------------------------------------------------------

_BIT_UFUNC = {"and": np.bitwise_and, "or": np.bitwise_or, "xor": np.bitwise_xor}


def _bit_neutral(op: str, dt: np.dtype):
    """Neutral element of a bitwise operator: all ones for ``&`` (true for Bool), zero for ``|`` and ``xor``."""
    if op == "and":
        return np.bool_(True) if dt == np.bool_ else dt.type(-1 if dt.kind == "i" else np.iinfo(dt).max)
    return dt.type(0)


def accumulate(op: str, A: np.ndarray, dims=None, init=None, inclusive: bool = True) -> np.ndarray:
    """``accumulate(op, A; dims, init)`` as the ROCArray methods define it.

    * eltype is preserved (``accumulate_eltype``); integer adds wrap.
    * ``dims=None`` is only legal for vectors (Base) -- there it scans the vector.
      ``dims > ndims(A)`` is an identity copy (test/core/rocarray_base.jl:204-213,
      ``(2,) => 2``).
    * ``init`` is folded in front: ``out[1] = op(init, A[1])``
      (test/core/rocarray_base.jl:198-200).
    * ``inclusive=False`` gives the exclusive scan seeded with ``init`` (AK keyword).

    Float inputs are scanned in Float64.
    """
    A = np.asarray(A)
    out_dt = accumulate_eltype(op, A.dtype)
    a = _wide(A, out_dt)
    if dims is None:
        if A.ndim != 1:
            raise ValueError("accumulate without dims needs a vector")
        axis = 0
    else:
        if dims < 1:
            raise ValueError("dims must be >= 1")
        axis = dims - 1
    if axis >= A.ndim:
        out = a.copy()                        # every element is a line of length 1: out[i] = op(init, A[i])
        if init is not None:
            seed = a.dtype.type(init)
            with np.errstate(over="ignore"):
                if op == "add":
                    out = out + seed
                elif op == "mul":
                    out = out * seed
                elif op in _BIT_UFUNC:
                    out = _BIT_UFUNC[op](out, seed)
                else:
                    out = (np.maximum if op == "max" else np.minimum)(out, seed)
        if not inclusive:
            if init is None and op in ("max", "min"):
                raise ValueError("exclusive max/min scans need init")
            neutral = _bit_neutral(op, a.dtype) if op in _BIT_UFUNC else a.dtype.type(0 if op == "add" else 1)
            out = np.full_like(a, neutral if init is None else a.dtype.type(init))
        return out
    with np.errstate(over="ignore"):
        if op == "add":
            inc = np.cumsum(a, axis=axis, dtype=a.dtype)
            neutral = a.dtype.type(0)
        elif op == "mul":
            inc = np.cumprod(a, axis=axis, dtype=a.dtype)
            neutral = a.dtype.type(1)
        elif op in ("max", "min"):
            fn = np.maximum if op == "max" else np.minimum
            inc = fn.accumulate(a, axis=axis)
            neutral = None
        elif op in _BIT_UFUNC:                      # accumulate(&, A), accumulate(|, A), accumulate(xor, A)
            inc = _BIT_UFUNC[op].accumulate(a, axis=axis)
            neutral = _bit_neutral(op, a.dtype)
        else:
            raise ValueError(f"unknown op {op!r}")
        seed = neutral if init is None else a.dtype.type(init)
        if init is not None:
            if op == "add":
                inc = inc + seed
            elif op == "mul":
                inc = inc * seed
            elif op in _BIT_UFUNC:
                inc = _BIT_UFUNC[op](inc, seed)
            else:
                inc = (np.maximum if op == "max" else np.minimum)(inc, seed)
        if inclusive:
            return inc
        if seed is None:
            raise ValueError("exclusive max/min scans need init")
        exc = np.empty_like(inc)
        sl_first = [slice(None)] * a.ndim
        sl_first[axis] = slice(0, 1)
        sl_rest = [slice(None)] * a.ndim
        sl_rest[axis] = slice(1, None)
        sl_src = [slice(None)] * a.ndim
        sl_src[axis] = slice(0, -1)
        exc[tuple(sl_first)] = seed
        exc[tuple(sl_rest)] = inc[tuple(sl_src)]
        return exc


def cumsum(A, dims=None):
    """``cumsum(::ROCArray; dims)`` -> AK.cumsum (src/kernels/accumulate.jl:7).

    Note: eltype-preserving (Int32 wraps), unlike Base.cumsum on Array which widens.
    """
    return accumulate("add", A, dims=dims)


def cumprod(A, dims=None):
    return accumulate("mul", A, dims=dims)


# ---------------------------------------------------------------------------
# findall  (src/kernels/indexing.jl:8-36: cumsum over the flattened Bool array, then
# scatter of CartesianIndices)
# ---------------------------------------------------------------------------

def findall(bools: np.ndarray) -> np.ndarray:
    """1-based indices of the true entries in column-major order.

    For vectors: Int64 vector of linear indices; for N-d: ``(count, N)`` Int64 array of
    Cartesian coordinates (``keytype(bools)``, indexing.jl:9).
    """
    b = np.asarray(bools).astype(bool)
    flat = b.reshape(-1, order="F")
    lin = np.nonzero(flat)[0].astype(np.int64)
    if b.ndim == 1:
        return lin + 1
    return np.stack(np.unravel_index(lin, b.shape, order="F"), axis=-1).astype(np.int64) + 1


def reverse(x: np.ndarray, start=None, stop=None, dims=None) -> np.ndarray:
    """``reverse(x)`` / ``reverse(x, start, stop)`` / ``reverse(x; dims)`` (src/kernels/reverse.jl:5-47, Base
    semantics): 1-based inclusive range for vectors, ``dims`` an Int, an iterable or None (= all)."""
    x = np.asarray(x)
    if start is not None:
        stop = x.shape[0] if stop is None else stop
        y = x.copy()
        y[start - 1:stop] = x[start - 1:stop][::-1]
        return y
    if dims is None:
        dims = range(1, x.ndim + 1)
    elif isinstance(dims, (int, np.integer)):
        dims = (dims,)
    idx = [slice(None)] * x.ndim
    for d in dims:
        idx[d - 1] = slice(None, None, -1)
    return x[tuple(idx)].copy()


def _isless_rank(x: np.ndarray) -> np.ndarray:
    """Unsigned integers that order like ``Base.isless`` on ``x`` (floats: -0.0 < 0.0, every NaN equal and last)."""
    x = np.asarray(x)
    if x.dtype.kind == "f":
        ut = {2: np.uint16, 4: np.uint32, 8: np.uint64}[x.dtype.itemsize]
        b = np.where(np.isnan(x), np.array(np.nan, dtype=x.dtype), x).view(ut)     # one NaN pattern for all NaNs
        sign = ut(1) << ut(8 * x.dtype.itemsize - 1)
        return np.where(b & sign != 0, ~b, b | sign)
    ut = np.dtype(f"u{x.dtype.itemsize}").type
    return x.view(ut) ^ (ut(1) << ut(8 * x.dtype.itemsize - 1))


def sortperm(x: np.ndarray, rev: bool = False) -> np.ndarray:
    """``sortperm(x; rev)`` (src/kernels/sorting.jl:3, Base semantics): 1-based, stable -- equal keys stay in
    index order, with ``rev=true`` too (Base reverses the ordering, not the result)."""
    r = _isless_rank(x)
    if rev:
        r = ~r
    return np.argsort(r, kind="stable").astype(np.int64) + 1


def sort(x: np.ndarray, rev: bool = False) -> np.ndarray:
    """``sort(x; rev)`` (src/kernels/sorting.jl:1): ``x[sortperm(x; rev)]``."""
    x = np.asarray(x)
    return x[sortperm(x, rev) - 1]


def permutedims(x: np.ndarray, perm) -> np.ndarray:
    """``permutedims(x, perm)`` (Base; 1-based perm): ``size(out, k) == size(x, perm[k])`` and
    ``out[i_perm[1], ..., i_perm[N]] == x[i_1, ..., i_N]``."""
    return np.transpose(np.asarray(x), [p - 1 for p in perm]).copy()


# ---------------------------------------------------------------------------
# broadcast   (src/broadcast.jl:3-35; kernel = GPUArrays _copyto!: dest[I] = bc[I],
# size-1 dims are extruded, trailing missing dims count as size 1)
# ---------------------------------------------------------------------------

def broadcast_shape(*shapes):
    """Julia's broadcast shape rule: align from the FIRST dim (not NumPy's last)."""
    nd = max((len(s) for s in shapes), default=0)
    out = []
    for d in range(nd):
        ext = 1
        for s in shapes:
            n = s[d] if d < len(s) else 1
            if n != 1:
                if ext != 1 and ext != n:
                    raise ValueError(f"DimensionMismatch: {shapes}")
                ext = n
        out.append(ext)
    return tuple(out)


def _jl_extrude(a, nd):
    """Pad a Julia-shaped array with trailing singleton dims so NumPy broadcasting
    (which aligns trailing dims) applies Julia's rule (which aligns leading dims)."""
    a = np.asarray(a)
    if a.ndim == 0:
        return a
    return a.reshape(a.shape + (1,) * (nd - a.ndim))


def broadcast_axpby_exp(a, x, y, w):
    """``z .= a .* x .+ y .* exp.(w)`` in Float64 (benchmark configuration 4a)."""
    x, y, w = (np.asarray(v, dtype=np.float64) for v in (x, y, w))
    nd = max(x.ndim, y.ndim, w.ndim)
    return float(a) * _jl_extrude(x, nd) + _jl_extrude(y, nd) * np.exp(_jl_extrude(w, nd))


def broadcast_rowcol(A, r, c):
    """``C .= A .+ r .* c`` with ``r`` of size 1xN and ``c`` of size Mx1 (config 4b)."""
    A, r, c = (np.asarray(v, dtype=np.float64) for v in (A, r, c))
    nd = max(A.ndim, r.ndim, c.ndim)
    return _jl_extrude(A, nd) + _jl_extrude(r, nd) * _jl_extrude(c, nd)


_UNARY = {
    "neg": np.negative, "abs": np.abs, "abs2": lambda v: v * v, "sqrt": np.sqrt,
    "exp": np.exp, "log": np.log, "sin": np.sin, "cos": np.cos, "tanh": np.tanh,
    "inv": lambda v: 1.0 / v, "identity": lambda v: v,
}
_BINARY = {
    "add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide,
    "max": np.maximum, "min": np.minimum, "pow": np.power,
}


def broadcast_eval(postfix, operands):
    """Evaluate a postfix broadcast program in Float64.

    ``postfix`` is a list of tokens: ``("arg", k)`` pushes operand k, a unary or binary
    op name pops its inputs and pushes the result, ``"fma"`` pops c, b, a and pushes
    ``a*b + c`` (Julia's ``muladd``).  Operands are Julia-shaped arrays or scalars.
    Mirrors what the fused kernel computes for ``dest .= f(args...)`` trees.
    """
    shapes = [np.shape(o) for o in operands]
    nd = max((len(s) for s in shapes), default=0)
    ops = [_jl_extrude(np.asarray(o, dtype=np.float64), nd) for o in operands]
    st = []
    for tok in postfix:
        if isinstance(tok, tuple):
            st.append(ops[tok[1]])
        elif tok in _UNARY:
            st.append(_UNARY[tok](st.pop()))
        elif tok in _BINARY:
            b = st.pop()
            a = st.pop()
            st.append(_BINARY[tok](a, b))
        elif tok == "fma":
            c = st.pop()
            b = st.pop()
            a = st.pop()
            st.append(a * b + c)
        else:
            raise ValueError(f"unknown token {tok!r}")
    assert len(st) == 1
    out_shape = broadcast_shape(*shapes)
    return np.broadcast_to(st[0], out_shape).copy()


# ---------------------------------------------------------------------------
# volumerhs   (perf/volumerhs.jl:42-176)
# ---------------------------------------------------------------------------

NQ = 5            # N + 1 with N = 4            (perf/volumerhs.jl:35,49)
NSTATE = 5        # rho, U, V, W, E             (perf/volumerhs.jl:22-24)
NVGEO = 14        # metric fields               (perf/volumerhs.jl:26-33)
_RHO, _U, _V, _W, _E = range(5)
_XIX, _ETAX, _ZETAX, _XIY, _ETAY, _ZETAY, _XIZ, _ETAZ, _ZETAZ, _MJ, _MJI, _X, _Y, _Z = range(14)
GDM1 = 0.4        # perf/volumerhs.jl:40
GRAV = 9.81       # perf/volumerhs.jl:39


def _fluxes(Q, vgeo, gravity):
    """Per-node metric-weighted fluxes F, G, H, shape (i, j, k, state, e).

    perf/volumerhs.jl:80-128.
    """
    rho, U, V, W, E = (Q[:, :, :, s, :] for s in (_RHO, _U, _V, _W, _E))
    MJ = vgeo[:, :, :, _MJ, :]
    z = vgeo[:, :, :, _Z, :]
    rinv = 1.0 / rho
    r2inv = 1.0 / (2.0 * rho)
    P = GDM1 * (E - (U * U + V * V + W * W) * r2inv - rho * gravity * z)     # :92
    fx = [U, rinv * U * U + P, rinv * U * V, rinv * U * W, rinv * U * (E + P)]  # :94-98
    fy = [V, rinv * V * U, rinv * V * V + P, rinv * V * W, rinv * V * (E + P)]  # :100-104
    fz = [W, rinv * W * U, rinv * W * V, rinv * W * W + P, rinv * W * (E + P)]  # :106-110
    out = []
    for (mx, my, mz) in ((_XIX, _XIY, _XIZ), (_ETAX, _ETAY, _ETAZ), (_ZETAX, _ZETAY, _ZETAZ)):
        ax, ay, az = vgeo[:, :, :, mx, :], vgeo[:, :, :, my, :], vgeo[:, :, :, mz, :]
        out.append(np.stack([MJ * (ax * fx[s] + ay * fy[s] + az * fz[s]) for s in range(5)], axis=3))
    return out  # F, G, H


def volumerhs(rhs, Q, vgeo, gravity, D):
    """Tensor-contraction restatement of ``volumerhs!``; returns the updated rhs.

    ``rhs[i,j,k,s,e] += MJI * ( sum_n D[n,i] F[n,j,k] + D[n,j] G[i,n,k] + D[n,k] H[i,j,n]
    - [s == W] MJ rho g )``  -- perf/volumerhs.jl:131-173.  All in Float64.
    Shapes: rhs, Q (5,5,5,5,nelem); vgeo (5,5,5,14,nelem); D (5,5).
    """
    rhs = np.asarray(rhs, dtype=np.float64)
    Q = np.asarray(Q, dtype=np.float64)
    vgeo = np.asarray(vgeo, dtype=np.float64)
    D = np.asarray(D, dtype=np.float64)
    g = float(gravity)
    F, G, H = _fluxes(Q, vgeo, g)
    acc = (np.einsum("ni,njkse->ijkse", D, F)
           + np.einsum("nj,inkse->ijkse", D, G)
           + np.einsum("nk,ijnse->ijkse", D, H))
    acc[:, :, :, _W, :] -= vgeo[:, :, :, _MJ, :] * Q[:, :, :, _RHO, :] * g      # :140
    return rhs + vgeo[:, :, :, _MJI, :][:, :, :, None, :] * acc                 # :166-173


def volumerhs_loops(rhs, Q, vgeo, gravity, D):
    """Literal loop-for-loop transcription of perf/volumerhs.jl:61-174 (Float64).

    Slow: meant for a handful of elements, as an independent check of ``volumerhs``.
    """
    rhs = np.array(rhs, dtype=np.float64)
    Q = np.asarray(Q, dtype=np.float64)
    vgeo = np.asarray(vgeo, dtype=np.float64)
    D = np.asarray(D, dtype=np.float64)
    g = float(gravity)
    nelem = Q.shape[4]
    for e in range(nelem):
        r = np.zeros((NQ, NQ, NQ, NSTATE))          # r_rhs*[k] per work-item (i, j)
        for k in range(NQ):
            sF = np.zeros((NQ, NQ, NSTATE))
            sG = np.zeros((NQ, NQ, NSTATE))
            for j in range(NQ):
                for i in range(NQ):
                    MJ = vgeo[i, j, k, _MJ, e]
                    xix, xiy, xiz = vgeo[i, j, k, _XIX, e], vgeo[i, j, k, _XIY, e], vgeo[i, j, k, _XIZ, e]
                    etx, ety, etz = vgeo[i, j, k, _ETAX, e], vgeo[i, j, k, _ETAY, e], vgeo[i, j, k, _ETAZ, e]
                    zex, zey, zez = vgeo[i, j, k, _ZETAX, e], vgeo[i, j, k, _ZETAY, e], vgeo[i, j, k, _ZETAZ, e]
                    z = vgeo[i, j, k, _Z, e]
                    U, V, W = Q[i, j, k, _U, e], Q[i, j, k, _V, e], Q[i, j, k, _W, e]
                    rho, E = Q[i, j, k, _RHO, e], Q[i, j, k, _E, e]
                    rinv = 1.0 / rho
                    r2inv = 1.0 / (2.0 * rho)
                    P = GDM1 * (E - (U ** 2 + V ** 2 + W ** 2) * r2inv - rho * g * z)
                    fx = (U, rinv * U * U + P, rinv * U * V, rinv * U * W, rinv * U * (E + P))
                    fy = (V, rinv * V * U, rinv * V * V + P, rinv * V * W, rinv * V * (E + P))
                    fz = (W, rinv * W * U, rinv * W * V, rinv * W * W + P, rinv * W * (E + P))
                    for s in range(NSTATE):
                        sF[i, j, s] = MJ * (xix * fx[s] + xiy * fy[s] + xiz * fz[s])
                        sG[i, j, s] = MJ * (etx * fx[s] + ety * fy[s] + etz * fz[s])
                        rH = MJ * (zex * fx[s] + zey * fy[s] + zez * fz[s])
                        for n in range(NQ):
                            r[i, j, n, s] += D[k, n] * rH                    # :131-138
                    r[i, j, k, _W] -= MJ * rho * g                            # :140
            for j in range(NQ):
                for i in range(NQ):
                    for n in range(NQ):
                        for s in range(NSTATE):
                            r[i, j, k, s] += D[n, i] * sF[n, j, s]            # :145-163
                            r[i, j, k, s] += D[n, j] * sG[i, n, s]
        for k in range(NQ):
            for j in range(NQ):
                for i in range(NQ):
                    MJI = vgeo[i, j, k, _MJI, e]
                    for s in range(NSTATE):
                        rhs[i, j, k, s, e] += MJI * r[i, j, k, s]              # :166-173
    return rhs


# ---------------------------------------------------------------------------
# deterministic inputs of the five benchmark configurations
# ---------------------------------------------------------------------------

def config_inputs(name: str, scale: float = 1.0):
    """Seeded inputs for the benchmark configurations (NumPy ``default_rng(seed)``).

    ``scale`` < 1 shrinks the problem (tests at sizes the oracle finishes in seconds).
    The same host buffer feeds both the device path and the oracle, so no cross-language
    RNG parity is needed.
    """
    def sz(n, lo=1):
        return max(lo, int(round(n * scale)))

    if name == "sum_f32":
        return {"x": np.random.default_rng(0).random(sz(1 << 24), dtype=np.float32)}
    if name == "sum_i32":
        return {"x": np.random.default_rng(0).integers(-1000, 1001, sz(1 << 24), dtype=np.int32)}
    if name == "dims_f32":
        n = sz(8192)
        return {"A": np.random.default_rng(1).standard_normal((n, n), dtype=np.float32)}
    if name == "cumsum_i32":
        return {"x": np.random.default_rng(2).integers(-1000, 1001, sz(1 << 27), dtype=np.int32)}
    if name == "cumsum_f32_dims1":
        return {"B": np.random.default_rng(2).random((sz(4096), sz(16384)), dtype=np.float32)}
    if name == "bcast_axpby_exp":
        n = sz(512)
        rng = np.random.default_rng(3)
        return {"a": np.float32(0.5),
                "x": rng.standard_normal((n, n, n), dtype=np.float32),
                "y": rng.standard_normal((n, n, n), dtype=np.float32),
                "w": rng.standard_normal((n, n, n), dtype=np.float32)}
    if name == "bcast_rowcol":
        n = sz(16384)
        rng = np.random.default_rng(3)
        u = lambda *s: (rng.random(s, dtype=np.float32) * 2 - 1).astype(np.float32)
        return {"A": u(n, n), "r": u(1, n), "c": u(n, 1)}
    if name == "volumerhs":
        ne = sz(4000)
        rng = np.random.default_rng(4)
        Q = (rng.random((NQ, NQ, NQ, NSTATE, ne), dtype=np.float32) + np.float32(0.5))
        vgeo = (rng.random((NQ, NQ, NQ, NVGEO, ne), dtype=np.float32) * np.float32(0.2)
                + np.float32(0.9))
        D = rng.random((NQ, NQ), dtype=np.float32)
        return {"Q": Q, "vgeo": vgeo, "D": D, "gravity": np.float32(GRAV),
                "rhs": np.zeros((NQ, NQ, NQ, NSTATE, ne), dtype=np.float32)}
    raise KeyError(name)
