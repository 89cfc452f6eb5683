"""GPU parity of reductions whose f is a closure (``mapreduce(x -> x + 1, +, A; dims)``, perf/array.jl:107-122;
``count(isodd, A)``, ``any(pred, A)``, ``findall(isodd, A)``, perf/array.jl:39-47) and of Bool-valued broadcasts.

mapreduce(f, op, A) is by definition mapreduce(identity, op, map(f, A)): the expected values apply f with NumPy in
Julia's element type (Int32 arithmetic wraps in both) and reduce the mapped array with the oracle.
Float32 sums: rtol 1e-5 against the Float64 host sum; integers, counts, Bools and indices bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL = 1e-5
SHAPES = [(512, 1000), (3, 100_000), (37, 41, 13), (1 << 20,), (5,), (1, 1)]


def _rng(seed):
    return np.random.default_rng(seed)


def _dims_for(shape):
    return [None] + list(range(1, len(shape) + 1)) + ([(1, 3)] if len(shape) == 3 else [])


@pytest.mark.parametrize("shape", SHAPES)
def test_mapreduce_plus_one_f32(rk, orc, shape):
    x = _rng(1).random(shape, dtype=np.float32)
    mapped = x + np.float32(1)
    for dims in _dims_for(shape):
        got = rk.mapreduce(lambda v: v + 1, "add", rk.ROCArray(x), dims=dims)
        want = orc.mapreduce("identity", "add", mapped, dims=dims)
        if dims is None:
            assert isinstance(got, np.float32)
            np.testing.assert_allclose(got, want.reshape(()), rtol=RTOL)
        else:
            assert got.dtype == np.float32 and got.dims == want.shape
            np.testing.assert_allclose(rk.Array(got), want, rtol=RTOL)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [np.int64, np.int32])
def test_mapreduce_plus_one_ints(rk, orc, shape, dtype):
    x = _rng(2).integers(-10, 11, shape).astype(dtype)
    for dims in _dims_for(shape):
        # x + 1 with an Int64 constant: Int32 elements map to Int64 (Julia's promotion), `+` keeps that type
        got = rk.mapreduce(lambda v: v + 1, "add", rk.ROCArray(x), dims=dims)
        want = orc.mapreduce("identity", "add", x.astype(np.int64) + 1, dims=dims)
        if dims is None:
            assert isinstance(got, np.int64) and got == want.reshape(())
        else:
            assert got.dtype == np.int64 and np.array_equal(rk.Array(got), want)
        # with a constant of the element type the mapped values, and `+`, stay in it
        one = dtype(1)
        got = rk.mapreduce(lambda v: v + one, "add", rk.ROCArray(x), dims=dims)
        want = orc.mapreduce("identity", "add", x + one, dims=dims)
        if dims is None:
            assert isinstance(got, dtype) and got == want.reshape(())
        else:
            assert got.dtype == dtype and np.array_equal(rk.Array(got), want)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int64, np.int32])
def test_one_operator_closures(rk, orc, dtype):
    """x + c, c + x, x - c, c - x, x * c, c * x under `+`: the library evaluates these without its interpreter (as
    x * m + a), which must not change a value -- integers bit-exact, floats within the tolerance of the sums, and the
    mapped values themselves (a reduction over a dim of extent 1; the sum starts from +0, so a -0 does not survive it,
    here as in the reference's neutral-element reductions) exactly."""
    rng = _rng(31)
    c = dtype(3) if np.dtype(dtype).kind == "i" else dtype(1.7)
    forms = [(lambda v: v + c, lambda x: x + c), (lambda v: c + v, lambda x: c + x), (lambda v: v - c, lambda x: x - c),
             (lambda v: c - v, lambda x: c - x), (lambda v: v * c, lambda x: x * c), (lambda v: c * v, lambda x: c * x)]
    for shape in ((100_003,), (300, 1001), (7, 33, 900)):
        x = (rng.integers(-50, 51, shape).astype(dtype) if np.dtype(dtype).kind == "i"
             else (rng.standard_normal(shape) * 3).astype(dtype))
        x.reshape(-1)[:4] = [0, -0.0, 1, -1] if np.dtype(dtype).kind == "f" else [0, 0, 1, -1]
        a = rk.ROCArray(x)
        for f, g in forms:
            mapped = g(x)
            for dims in _dims_for(shape):
                got = rk.mapreduce(f, "add", a, dims=dims)
                want = orc.mapreduce("identity", "add", mapped, dims=dims)
                got = np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape)
                if np.dtype(dtype).kind == "i":
                    assert got.dtype == want.dtype and np.array_equal(got, want)
                else:
                    np.testing.assert_allclose(got, want, rtol=RTOL, atol=1e-3 if dtype == np.float32 else 1e-9)
            # every output is one mapped element: the value of f itself
            one = rk.ROCArray(x.reshape(shape + (1,)))
            got = rk.Array(rk.mapreduce(f, "add", one, dims=len(shape) + 1)).reshape(shape)
            assert got.dtype == mapped.dtype and np.array_equal(got, mapped)


def test_int32_maps_wrap_like_julia(rk, orc):
    x = _rng(3).integers(-2**31, 2**31, (300, 1001)).astype(np.int32)
    with np.errstate(over="ignore"):
        sq = x * x                                       # wraps in Int32
        for dims in (None, 1, 2):
            a = rk.ROCArray(x)
            got = rk.mapreduce(lambda v: v * v, "add", a, dims=dims)              # Int32 sum of Int32 squares
            want = orc.mapreduce("identity", "add", sq, dims=dims)
            assert np.array_equal(np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape), want)
            got = rk.sum(lambda v: v * v, a, dims=dims)                           # add_sum widens the wrapped squares
            want = orc.mapreduce("identity", "add_sum", sq, dims=dims)
            assert np.array_equal(np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape), want)
            got = rk.count(lambda v: v * v > 0, a, dims=dims)                     # the comparison sees the wrapped value
            want = orc.mapreduce("identity", "add_sum", sq > 0, dims=dims)
            assert np.array_equal(np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape), want)
            got = rk.maximum(lambda v: rk.broadcast.max_(v * v, v + v), a, dims=dims)
            want = orc.mapreduce("identity", "max", np.maximum(sq, x + x), dims=dims)
            assert np.array_equal(np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape), want)


@pytest.mark.parametrize("dtype", [np.int64, np.int32, np.float32, np.float64, np.bool_])
def test_count_any_all_with_predicates(rk, orc, dtype):
    shape = (129, 517)
    rng = _rng(4)
    if dtype == np.bool_:
        x = rng.random(shape) < 0.4
        preds = [(lambda v: ~v, ~x)]
    elif np.dtype(dtype).kind == "i":
        x = rng.integers(-10, 11, shape).astype(dtype)
        preds = [(lambda v: rk.isodd(v), x % 2 != 0), (lambda v: rk.iseven(v + 1), (x + 1) % 2 == 0),
                 (lambda v: (v > -3) & (v <= 4), (x > -3) & (x <= 4)), (lambda v: v == 11, x == 11), (lambda v: v != 11, x != 11)]
    else:
        x = rng.standard_normal(shape).astype(dtype)
        x[5, 7] = np.nan
        half = dtype(0.5)
        preds = [(lambda v: v > half, x > half), (lambda v: rk.isnan(v), np.isnan(x)), (lambda v: (v < -half) | (v >= half), (x < -half) | (x >= half)),
                 (lambda v: v * v < half, x * x < half), (lambda v: v > 100, x > 100), (lambda v: v == v, x == x)]
    a = rk.ROCArray(x)
    for pred, mask in preds:
        for dims in (None, 1, 2, (1, 2)):
            ax = None if dims is None else tuple(d - 1 for d in ((dims,) if isinstance(dims, int) else dims))
            got = rk.count(pred, a, dims=dims)
            want = mask.sum(axis=ax, keepdims=dims is not None, dtype=np.int64)
            if dims is None:
                assert isinstance(got, np.int64) and got == want
            else:
                assert got.dtype == np.int64 and np.array_equal(rk.Array(got), want)
            for fn, ref in ((rk.any, np.any), (rk.all, np.all)):
                got = fn(pred, a, dims=dims)
                want = ref(mask, axis=ax, keepdims=dims is not None)
                if dims is None:
                    assert isinstance(got, bool) and got == bool(want)
                else:
                    assert got.dtype == np.bool_ and np.array_equal(rk.Array(got), want)


def test_sum_maximum_minimum_of_closures(rk, orc):
    x = _rng(5).standard_normal((257, 1025)).astype(np.float32)
    two, half = np.float32(2), np.float32(0.5)
    a = rk.ROCArray(x)
    cases = [
        (rk.sum, lambda v: v * v - two * v + half, x * x - two * x + half, "add_sum"),
        (rk.sum, lambda v: rk.broadcast.exp(-(v * v)), np.exp(-(x * x)), "add_sum"),
        (rk.sum, lambda v: rk.ifelse(v > 0, v, half * v), np.where(x > 0, x, half * x), "add_sum"),
        (rk.maximum, lambda v: rk.broadcast.abs_(v - half), np.abs(x - half), "max"),
        (rk.minimum, lambda v: rk.broadcast.muladd(v, v, half), x * x + half, "min"),
        (rk.prod, lambda v: np.float32(1) + np.float32(1e-4) * v, np.float32(1) + np.float32(1e-4) * x, "mul_prod"),
    ]
    for fn, f, mapped, op in cases:
        for dims in (None, 1, 2):
            got = fn(f, a, dims=dims)
            want = orc.mapreduce("identity", op, mapped.astype(np.float32), dims=dims)
            got = np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape)
            # a Float32 product of 263k factors near 1 drifts by ~1e-3 in any evaluation order (a lane-wise NumPy
            # Float32 product of the same factors does too); the exact check of prod is the +-1 case below
            np.testing.assert_allclose(got, want, rtol=5e-3 if op == "mul_prod" else 2e-5, atol=1e-3 if op == "add_sum" else 0)
    k = _rng(8).integers(-10, 11, (257, 1025))
    for dims in (None, 1, 2):
        got = rk.prod(lambda v: rk.ifelse(rk.isodd(v), -1, 1), rk.ROCArray(k), dims=dims)
        want = orc.mapreduce("identity", "mul_prod", np.where(k % 2 != 0, -1, 1), dims=dims)
        assert np.array_equal(np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape), want)
    xd = x.astype(np.float64)
    got = rk.sum(lambda v: v * v + 0.25, rk.ROCArray(xd))                  # Float64 elements take Python floats
    assert isinstance(got, np.float64)
    np.testing.assert_allclose(got, (xd * xd + 0.25).sum(), rtol=1e-12)


def test_findall_and_findfirst_with_predicates(rk, orc):
    x = _rng(6).integers(-10, 11, (512, 1000))
    a = rk.ROCArray(x)
    v = a.reshape(x.size)
    flat = x.reshape(-1, order="F")
    got = rk.Array(rk.findall(lambda e: rk.isodd(e), v))
    assert np.array_equal(got, np.nonzero(flat % 2 != 0)[0] + 1)
    got2 = rk.Array(rk.findall(lambda e: e == 7, a))                          # CartesianIndex columns
    want = orc.findall(x == 7)
    assert np.array_equal(got2, want.T)
    assert rk.findfirst(lambda e: rk.isodd(e), v) == int(np.nonzero(flat % 2 != 0)[0][0]) + 1
    assert rk.findfirst(lambda e: e > 10, v) is None
    i, j = rk.findfirst(lambda e: e == -10, a)
    assert flat.tolist().index(-10) == (i - 1) + (j - 1) * 512


def test_bool_valued_broadcasts(rk):
    rng = _rng(7)
    x = rng.standard_normal((130, 257)).astype(np.float32)
    y = rng.standard_normal((130, 1)).astype(np.float32)
    k = rng.integers(-5, 6, (130, 257)).astype(np.int32)
    x[3, 3] = np.nan
    X, Y, K = rk.ROCArray(x), rk.ROCArray(y), rk.ROCArray(k)
    lz = rk.lazy
    cases = [
        (lz(X) > lz(Y), x > y), (lz(X) <= 0, x <= 0), (lz(X) == lz(X), x == x), (lz(X) != lz(Y), x != y),
        ((lz(X) > 0) & (lz(Y) < 0), (x > 0) & (y < 0)), ((lz(X) > 1) | ~(lz(Y) < 0), (x > 1) | ~(y < 0)),
        (rk.isnan(lz(X)), np.isnan(x)), (rk.isodd(lz(K)), k % 2 != 0), (rk.iseven(lz(K) * 3 + 1), (k * 3 + 1) % 2 == 0),
        (lz(K) >= 2, k >= 2),
    ]
    for bc, want in cases:
        got = rk.materialize(bc)
        assert got.dtype == np.bool_ and np.array_equal(rk.Array(got), want)
    got = rk.materialize(rk.ifelse(lz(X) > lz(Y), lz(X), lz(Y) * np.float32(2)))
    assert got.dtype == np.float32
    np.testing.assert_array_equal(rk.Array(got), np.where(x > y, x, y * np.float32(2)))
    got = rk.materialize(rk.ifelse(rk.isodd(lz(K)), lz(K), -lz(K)))            # Int32 in, Int32 out
    assert got.dtype == np.int32 and np.array_equal(rk.Array(got), np.where(k % 2 != 0, k, -k))
    big = rng.integers(2**30, 2**31, (1000,)).astype(np.int32)
    with np.errstate(over="ignore"):
        got = rk.materialize((rk.lazy(rk.ROCArray(big)) + rk.lazy(rk.ROCArray(big))) > 0)   # the Int32 sum wraps below zero
        assert np.array_equal(rk.Array(got), (big + big) > 0)


def test_closures_outside_the_kernel_set_map_first(rk, orc):
    """Closures the reduction kernels do not interpret take two kernels (broadcast, then reduce): same results."""
    x = _rng(9).standard_normal((33, 1000)).astype(np.float32)
    y = _rng(10).standard_normal((33, 1000)).astype(np.float32)
    a, b = rk.ROCArray(x), rk.ROCArray(y)
    for dims in (None, 1, 2):
        got = rk.sum(lambda v: rk.broadcast.sin(v) * rk.broadcast.cos(v), a, dims=dims)        # trigonometry
        want = orc.mapreduce("identity", "add_sum", (np.sin(x.astype(np.float64)) * np.cos(x.astype(np.float64))).astype(np.float32), dims=dims)
        np.testing.assert_allclose(np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape), want, rtol=1e-4, atol=1e-3)
        got = rk.sum(lambda v: (v - rk.lazy(b)) * (v - rk.lazy(b)), a, dims=dims)              # captures an array
        want = orc.mapreduce("identity", "add_sum", (x - y) * (x - y), dims=dims)
        np.testing.assert_allclose(np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape), want, rtol=2e-5, atol=1e-3)
        got = rk.sum(lambda v: v * 0.5, a, dims=dims)                                           # Float64 constant: a Float64 sum
        want = (x.astype(np.float64) * 0.5).sum(axis=None if dims is None else dims - 1, keepdims=dims is not None)
        assert (got.dtype if dims is not None else np.asarray(got).dtype) == np.float64
        np.testing.assert_allclose(np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape), want, rtol=1e-12, atol=1e-9)
        got = rk.sum(lambda v: ((((v + 1) * v + 2) * v + 3) * v + 4) * v + 5, a, dims=dims)   # five constants
        x64 = x.astype(np.float64)
        want = (((((x64 + 1) * x64 + 2) * x64 + 3) * x64 + 4) * x64 + 5).sum(axis=None if dims is None else dims - 1, keepdims=dims is not None)
        np.testing.assert_allclose(np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape), want, rtol=1e-4, atol=1e-2)


def test_unsupported_closures(rk):
    x = rk.ROCArray(np.ones((4, 4), dtype=np.float32))
    with pytest.raises(rk.UnsupportedError):
        rk.mapreduce(lambda v: rk.isodd(v), "add", x)                            # isodd of a Float32
    with pytest.raises(TypeError):
        rk.count(lambda v: v + 1, x)                                             # not a predicate
    with pytest.raises(rk.UnsupportedError):
        rk.sum(lambda v: v if v > 0 else -v, x)                                  # a branch on the value: ifelse can be traced, `if` cannot
    with pytest.raises(rk.UnsupportedError):
        rk.materialize(rk.lazy(x) if rk.lazy(x) > 0 else -rk.lazy(x))
