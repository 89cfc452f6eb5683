"""GPU parity of mapreduce / sum / maximum / findmax against the oracle, through the C ABI.

Tolerances (stated by the task): Float32 sums rtol 1e-5 against a Float64 host sum; integer results and
findmax values + indices bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL_SUM = 1e-5


def _rng(seed):
    return np.random.default_rng(seed)


@pytest.mark.parametrize("n", [1, 2, 3, 63, 64, 65, 255, 256, 257, 1000, 4095, 4096, 4097, 65536, 100_003, 1 << 20, (1 << 22) + 7])
def test_sum_f32_sizes(rk, orc, n):
    x = _rng(n).random(n, dtype=np.float32)
    got = rk.sum(rk.ROCArray(x))
    assert isinstance(got, np.float32)
    np.testing.assert_allclose(got, orc.sum_(x), rtol=RTOL_SUM)


@pytest.mark.parametrize("n", [1, 5, 64, 1000, 4097, 1 << 18, (1 << 21) + 3])
def test_sum_i32_widens_and_is_exact(rk, orc, n):
    x = _rng(n).integers(-1000, 1001, n, dtype=np.int32)
    got = rk.sum(rk.ROCArray(x))
    assert isinstance(got, np.int64)
    assert got == orc.sum_(x)


def test_sum_i32_needs_int64(rk):
    # 2^22 * 1000 > 2^31: an Int32 accumulator would wrap
    x = np.full(1 << 22, 1000, dtype=np.int32)
    assert rk.sum(rk.ROCArray(x)) == (1 << 22) * 1000


def test_config1_full_size(rk, orc):
    x = orc.config_inputs("sum_f32")["x"]
    np.testing.assert_allclose(rk.sum(rk.ROCArray(x)), np.sum(x, dtype=np.float64), rtol=RTOL_SUM)
    xi = orc.config_inputs("sum_i32")["x"]
    assert rk.sum(rk.ROCArray(xi)) == int(xi.astype(np.int64).sum())


def test_reference_doctests(rk):
    # docs/src/usage/arrays.md:85-89
    assert rk.sum(rk.ROCArray(np.arange(1, 101, dtype=np.int64))) == 5050
    assert rk.mapreduce(rk.abs2, rk.add, rk.ROCArray(np.arange(1, 5, dtype=np.int64))) == 30
    # test/hip_rocarray/multi_gpu.jl:45
    assert rk.sum(rk.ROCArray(np.ones(16, dtype=np.int64))) == 16


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
@pytest.mark.parametrize("op", ["add", "mul", "max", "min"])
def test_ops_and_dtypes_full(rk, orc, dtype, op):
    rng = _rng(7)
    n = 5000
    if op == "mul":
        x = (rng.random(n) * 0.02 + 0.99).astype(dtype) if np.dtype(dtype).kind == "f" else rng.integers(-3, 4, n).astype(dtype)
    else:
        x = (rng.standard_normal(n) * 100).astype(dtype)
    got = rk.mapreduce(rk.identity, op, rk.ROCArray(x))
    want = orc.mapreduce("identity", op, x)
    assert got.dtype == orc.reduce_eltype(op, dtype)      # the oracle itself accumulates floats in Float64
    if np.dtype(dtype).kind == "f" and op in ("add", "mul"):
        np.testing.assert_allclose(got, want, rtol=1e-5 if dtype == np.float32 else 1e-12, atol=1e-3 if op == "add" else 0)
    else:
        assert got == want


@pytest.mark.parametrize("f", ["identity", "abs2", "abs"])
def test_maps(rk, orc, f):
    x = _rng(3).standard_normal(70_001).astype(np.float32)
    np.testing.assert_allclose(rk.mapreduce(f, "add", rk.ROCArray(x)), orc.mapreduce(f, "add", x), rtol=RTOL_SUM, atol=1e-3)
    xi = _rng(4).integers(-50, 50, 70_001, dtype=np.int32)
    assert rk.mapreduce(f, "add_sum", rk.ROCArray(xi)) == orc.mapreduce(f, "add_sum", xi)


def test_bool_count(rk, orc):
    b = _rng(5).random(100_000) < 0.3
    assert rk.sum(rk.ROCArray(b)) == int(b.sum())
    assert rk.count(rk.ROCArray(b)) == int(b.sum())


def test_unaligned_view(rk, orc):
    x = _rng(6).random(100_000, dtype=np.float32)
    d = rk.ROCArray(x)
    for first, last in [(2, 100_000), (3, 99_999), (4, 77_777), (1, 5)]:
        np.testing.assert_allclose(rk.sum(d.view_range(first, last)), orc.sum_(x[first - 1:last]), rtol=RTOL_SUM)


def test_init_is_folded_in(rk, orc):
    x = _rng(8).random(10_000, dtype=np.float32)
    np.testing.assert_allclose(rk.mapreduce("identity", "add", rk.ROCArray(x), init=np.float32(100)), orc.sum_(x) + 100, rtol=RTOL_SUM)


def test_empty(rk):
    e = rk.ROCArray(np.zeros(0, dtype=np.float32))
    assert rk.sum(e) == 0
    with pytest.raises(ValueError):
        rk.maximum(e)


def test_maximum_nan_and_signed_zero(rk):
    x = np.array([1, -0.0, 0.0, -5], dtype=np.float32)
    assert rk.maximum(rk.ROCArray(np.array([-0.0, 0.0], dtype=np.float32))) == 0 and not np.signbit(rk.maximum(rk.ROCArray(np.array([-0.0, 0.0], dtype=np.float32))))
    assert np.signbit(rk.minimum(rk.ROCArray(np.array([0.0, -0.0], dtype=np.float32))))
    y = np.concatenate([_rng(0).random(5000, dtype=np.float32), [np.nan], _rng(1).random(5000, dtype=np.float32)]).astype(np.float32)
    assert np.isnan(rk.maximum(rk.ROCArray(y))) and np.isnan(rk.minimum(rk.ROCArray(y)))
    assert rk.maximum(rk.ROCArray(x)) == 1 and rk.minimum(rk.ROCArray(x)) == -5


# ---- dimensional reductions ---------------------------------------------------------------------------
SHAPES_DIMS = [
    ((7,), 1), ((5, 3), 1), ((5, 3), 2), ((3, 4, 5), 1), ((3, 4, 5), 2), ((3, 4, 5), 3), ((1, 70, 50, 20), 3),
    ((64, 64), 1), ((64, 64), 2), ((100, 1000), 1), ((100, 1000), 2), ((1000, 100), 1), ((1000, 100), 2),
    ((512, 1000), 1), ((512, 1000), 2), ((3, 100_000), 1), ((3, 100_000), 2), ((100_000, 3), 1), ((100_000, 3), 2),
    ((257, 129, 5), 2), ((8, 4096, 3), 2), ((2, 3, 4, 5, 6), 4), ((33, 65), (1, 2)), ((6, 7, 8), (1, 3)),
    ((6, 7, 8), (2, 3)), ((6, 7, 8), (1, 2)), ((40, 50), 3),
]


@pytest.mark.parametrize("shape,dims", SHAPES_DIMS)
def test_abs2_sum_dims(rk, orc, shape, dims):
    A = _rng(11).standard_normal(shape).astype(np.float32)
    got = rk.mapreduce(rk.abs2, rk.add, rk.ROCArray(A), dims=dims)
    want = orc.mapreduce("abs2", "add", A, dims=dims)
    assert got.dims == want.shape
    np.testing.assert_allclose(rk.Array(got), want, rtol=RTOL_SUM)


@pytest.mark.parametrize("shape,dims", SHAPES_DIMS)
def test_sum_dims_i32_exact(rk, orc, shape, dims):
    A = _rng(12).integers(-1000, 1001, shape).astype(np.int32)
    got = rk.sum(rk.ROCArray(A), dims=dims)
    want = orc.sum_(A, dims=dims)
    assert got.dtype == np.int64 and got.dims == want.shape
    assert np.array_equal(rk.Array(got), want)


@pytest.mark.parametrize("shape,dims", SHAPES_DIMS)
def test_maximum_dims_exact(rk, orc, shape, dims):
    A = _rng(13).standard_normal(shape).astype(np.float32)
    assert np.array_equal(rk.Array(rk.maximum(rk.ROCArray(A), dims=dims)), orc.maximum(A, dims=dims))
    assert np.array_equal(rk.Array(rk.minimum(rk.ROCArray(A), dims=dims)), orc.minimum(A, dims=dims))


def _check_findminmax(rk, orc, A, dims):
    dA = rk.ROCArray(A)
    for gpu, cpu in ((rk.findmax, orc.findmax), (rk.findmin, orc.findmin)):
        gv, gi = gpu(dA, dims=dims)
        ov, oi = cpu(A, dims=dims)
        if dims is None:
            assert (gv == ov or (np.isnan(gv) and np.isnan(ov))) and gi == oi
            assert np.signbit(gv) == np.signbit(ov)
        else:
            assert np.array_equal(rk.Array(gv), ov, equal_nan=True)
            assert np.array_equal(np.signbit(rk.Array(gv)), np.signbit(ov))
            assert np.array_equal(np.moveaxis(rk.Array(gi), 0, -1), oi)


@pytest.mark.parametrize("shape,dims", SHAPES_DIMS + [((1000,), None), ((50, 60), None), ((1 << 20,), None)])
def test_findminmax_dims(rk, orc, shape, dims):
    rng = _rng(14)
    # few distinct values -> many ties, so the first-index rule is exercised
    A = rng.integers(-4, 5, shape).astype(np.float32)
    _check_findminmax(rk, orc, A, dims)
    _check_findminmax(rk, orc, rng.standard_normal(shape).astype(np.float32), dims)


@pytest.mark.parametrize("shape", [(64, 50_000), (100, 30_001), (128, 20_000), (65, 40_000, 3), (96, 5_000, 2), (127, 9_999), (64, 17), (72, 3_000, 5)])
def test_findminmax_along_long_lines_behind_short_rows(rk, orc, shape):
    """findmax / findmin(A; dims=2) with rows of 64 .. 128 elements (Float64, Int64: 64): several rows go into one load
    instruction, a group of lanes each, and the groups are folded across the lanes at the end.  Few distinct values, so
    that ties between rows of different lane groups decide by the first-index rule; the neighbouring shapes take the
    plain kernels."""
    rng = _rng(sum(shape))
    for dtype in (np.float32, np.float64, np.int32, np.int64):
        A = rng.integers(-3, 4, shape).astype(dtype)
        _check_findminmax(rk, orc, A, 2)
    A = rng.standard_normal(shape).astype(np.float32)
    A[shape[0] // 2, shape[1] // 3] = np.nan
    _check_findminmax(rk, orc, A, 2)


def test_findmax_nan_and_zero_rules(rk, orc):
    A = np.array([[1, np.nan, -0.0, 3], [np.nan, 2, 0.0, 3], [5, np.nan, -0.0, -np.inf]], dtype=np.float32)
    for dims in (1, 2, None):
        _check_findminmax(rk, orc, A, dims)
    big = _rng(15).standard_normal((300, 70)).astype(np.float32)
    big[17, 3] = np.nan
    big[200, 3] = np.nan
    big[5, 9] = np.nan
    for dims in (1, 2, None):
        _check_findminmax(rk, orc, big, dims)


@pytest.mark.parametrize("dtype", [np.float64, np.int32, np.int64])
def test_findmax_other_dtypes(rk, orc, dtype):
    A = _rng(16).integers(-100, 100, (65, 130)).astype(dtype)
    for dims in (1, 2, None):
        _check_findminmax(rk, orc, A, dims)


def test_config2_full_size(rk, orc):
    A = orc.config_inputs("dims_f32")["A"]
    dA = rk.ROCArray(A)
    A64 = A.astype(np.float64)
    for d in (1, 2):
        got = rk.Array(rk.mapreduce(rk.abs2, rk.add, dA, dims=d))
        np.testing.assert_allclose(got, (A64 * A64).sum(axis=d - 1, keepdims=True), rtol=RTOL_SUM)
    v, i = rk.findmax(dA, dims=1)
    v, i = rk.Array(v), rk.Array(i)
    assert np.array_equal(v, A.max(axis=0, keepdims=True))
    assert np.array_equal(i[0, 0, :], A.argmax(axis=0) + 1)
    assert np.array_equal(i[1, 0, :], np.arange(1, A.shape[1] + 1))


def test_mapreducedim_returns_R_and_pads_dims(rk):
    # test/core/rocarray_base.jl:263-267: R of size (3, 2) reduces A of size (3, 2, 10) over dim 3
    A = _rng(17).random((3, 2, 10), dtype=np.float32)
    R = rk.zeros(np.float32, 3, 2)
    out = rk.mapreducedim_(rk.identity, rk.add, R, rk.ROCArray(A))
    assert out is R
    np.testing.assert_allclose(rk.Array(R), A.astype(np.float64).sum(axis=2), rtol=RTOL_SUM)
    with pytest.raises(rk.DimensionMismatch):
        rk.mapreducedim_(rk.identity, rk.add, rk.zeros(np.float32, 2, 2), rk.ROCArray(A))


def test_repeated_calls_reuse_clean_workspace(rk, orc):
    # the multi-workgroup kernels must leave their tickets clean
    x = _rng(18).random(1 << 21, dtype=np.float32)
    d = rk.ROCArray(x)
    first = rk.sum(d)
    for _ in range(5):
        assert rk.sum(d) == first          # deterministic: same launch geometry, fixed combine order
    A = _rng(19).standard_normal((2048, 512)).astype(np.float32)
    dA = rk.ROCArray(A)
    r0 = rk.Array(rk.sum(dA, dims=2))
    for _ in range(3):
        assert np.array_equal(rk.Array(rk.sum(dA, dims=2)), r0)


@pytest.mark.parametrize("shape", [(1,), (1000,), (1 << 20,), (300, 70), (70, 300), (17, 5, 33)])
def test_any_all_findfirst_bool(rk, orc, shape):
    # Bool reductions run on the bytes: any = max, all = min, findfirst = argmax with ties to the smallest index
    rng = _rng(40)
    for p in (0.0, 1e-4, 0.5, 1.0):
        b = rng.random(shape) < p
        d = rk.ROCArray(b)
        assert rk.any(d) == bool(b.any()) and rk.all(d) == bool(b.all())
        flat = b.reshape(-1, order="F")
        want = None if not flat.any() else int(np.argmax(flat)) + 1
        got = rk.findfirst(d)
        if want is None or b.ndim == 1:
            assert got == want
        else:
            assert tuple(got) == tuple(int(i) + 1 for i in np.unravel_index(want - 1, b.shape, order="F"))
        for dims in range(1, b.ndim + 1):
            ra, rl = rk.any(d, dims=dims), rk.all(d, dims=dims)
            assert ra.dtype == np.bool_ and rl.dtype == np.bool_
            assert np.array_equal(rk.Array(ra), b.any(axis=dims - 1, keepdims=True))
            assert np.array_equal(rk.Array(rl), b.all(axis=dims - 1, keepdims=True))
    one = np.zeros(shape, dtype=bool)
    one[(-1,) * one.ndim] = True                                  # the last element in column-major order too
    got = rk.findfirst(rk.ROCArray(one))
    assert (got if one.ndim == 1 else int(np.ravel_multi_index(tuple(i - 1 for i in got), one.shape, order="F")) + 1) == one.size


@pytest.mark.parametrize("dtype", [np.uint32, np.uint64, np.uint8])
def test_unsigned_reductions(rk, orc, dtype):
    rng = _rng(41)
    info = np.iinfo(dtype)
    for shape, dims in [((100_003,), None), ((300, 70), 1), ((300, 70), 2), ((17, 5, 33), (1, 3))]:
        A = rng.integers(0, info.max, shape, dtype=dtype, endpoint=True)
        d = rk.ROCArray(A)
        s = rk.sum(d, dims=dims)                                       # add_sum widens UInt8 / UInt32 to UInt64
        want = orc.mapreduce("identity", "add_sum", A, dims=dims)
        if dims is None:
            assert s == want and np.asarray(s).dtype == np.uint64
        else:
            assert s.dtype == np.uint64 and np.array_equal(rk.Array(s), want)
        if dtype == np.uint8:
            continue
        assert np.array_equal(np.asarray(rk.Array(rk.maximum(d, dims=dims)) if dims else rk.maximum(d)), orc.maximum(A, dims=dims))
        assert np.array_equal(np.asarray(rk.Array(rk.minimum(d, dims=dims)) if dims else rk.minimum(d)), orc.minimum(A, dims=dims))
        if dims in (None, 1, 2):
            _check_findminmax(rk, orc, A, dims)
        # plain + keeps the eltype and wraps
        r = rk.mapreduce(rk.identity, rk.add, d, dims=dims)
        with np.errstate(over="ignore"):
            want = A.sum(dtype=dtype) if dims is None else A.sum(axis=tuple(x - 1 for x in ((dims,) if isinstance(dims, int) else dims)), keepdims=True, dtype=dtype)
        assert np.array_equal(np.asarray(r if dims is None else rk.Array(r)), want)


def test_argmax_argmin_extrema(rk, orc):
    rng = _rng(41)
    A = rng.integers(-50, 51, (37, 1001)).astype(np.float32)
    dA = rk.ROCArray(A)
    assert rk.argmax(dA) == orc.findmax(A)[1] and rk.argmin(dA) == orc.findmin(A)[1]
    for dims in (1, 2):
        assert np.array_equal(np.moveaxis(rk.Array(rk.argmax(dA, dims=dims)), 0, -1), orc.findmax(A, dims=dims)[1])
        assert np.array_equal(np.moveaxis(rk.Array(rk.argmin(dA, dims=dims)), 0, -1), orc.findmin(A, dims=dims)[1])
        lo, hi = rk.extrema(dA, dims=dims)
        assert np.array_equal(rk.Array(lo), A.min(axis=dims - 1, keepdims=True)) and np.array_equal(rk.Array(hi), A.max(axis=dims - 1, keepdims=True))
    assert rk.extrema(dA) == (A.min(), A.max())
    lo, hi = rk.extrema(lambda v: v * v, dA)
    assert (lo, hi) == ((A * A).min(), (A * A).max())


@pytest.mark.parametrize("shape,dims", [((1000,), None), ((257, 129), 1), ((257, 129), 2), ((33, 65, 17), (1, 3)), ((1 << 20,), None), ((8, 100_000), 2)])
def test_float16_reductions(rk, orc, shape, dims):
    """Float16 arrays: f applied in Float16, accumulated in Float32, rounded once to Float16.  Sums within one Float16
    rounding (2^-11 relative) plus the Float32 accumulation error of the Float64 result; max / min / findmax exact."""
    rng = _rng(61)
    x = rng.standard_normal(shape).astype(np.float16)
    dx = rk.ROCArray(x)
    x64 = x.astype(np.float64)
    ax = None if dims is None else tuple(d - 1 for d in ((dims,) if isinstance(dims, int) else dims))
    for f, mapped in (("identity", x64), ("abs2", (x * x).astype(np.float64)), ("abs", np.abs(x64))):
        got = rk.mapreduce(f, "add_sum", dx, dims=dims)
        want = mapped.sum(axis=ax, keepdims=dims is not None)
        mag = np.abs(mapped).sum(axis=ax, keepdims=dims is not None)
        got = np.asarray(got if dims is None else rk.Array(got))
        assert got.dtype == np.float16
        got = got.astype(np.float64).reshape(want.shape)
        with np.errstate(over="ignore"):
            over = np.isinf(want.astype(np.float16))              # beyond 65504: Inf, as in Julia
        assert np.array_equal(np.isinf(got), over)
        assert np.all(over | (np.abs(got - want) <= 2.0**-10 * np.abs(want) + 1e-6 * mag + 1e-7))
        for op, ref in (("max", np.max), ("min", np.min)):
            got = rk.mapreduce(f, op, dx, dims=dims)
            got = np.asarray(got if dims is None else rk.Array(got))
            want = ref(mapped, axis=ax, keepdims=dims is not None).astype(np.float16)
            assert got.dtype == np.float16 and np.array_equal(got.reshape(want.shape), want)
    if dims is None or isinstance(dims, int):
        _check_findminmax(rk, orc, rng.integers(-4, 5, shape).astype(np.float16), dims)
        _check_findminmax(rk, orc, x, dims)
    init = rk.mapreduce("identity", "add", dx, dims=dims, init=np.float16(2.5))
    init = np.asarray(init if dims is None else rk.Array(init)).astype(np.float64)
    want = x64.sum(axis=ax, keepdims=dims is not None) + 2.5
    assert np.all(np.abs(init.reshape(want.shape) - want) <= 2.0**-10 * np.abs(want) + 1e-6 * np.abs(x64).sum(axis=ax, keepdims=dims is not None) + 1e-7)


@pytest.mark.parametrize("shape,dims", [((3, 100_000), 2), ((7, 52_429, 5), 2), ((2, 3, 200_001), 3), ((63, 4099), 2), ((5, 5, 5, 5, 2000), 5),
                                        ((2, 3, 200_001), (1, 3)), ((5, 5, 5, 5, 2000), (1, 5)), ((33, 1025, 2), 2), ((16, 1024), 2), ((2, 1_000_003), 2)])
def test_long_lines_with_a_narrow_inner_extent(rk, orc, shape, dims):
    """1 < inner < 64 along a long reduced dim (sum(A; dims=2) of a 3 x N array), alone and as the first fold of a
    reduction over non-adjacent dims."""
    rng = _rng(71)
    for dtype in (np.float32, np.int32, np.int64, np.float64):
        x = rng.integers(-1000, 1001, shape).astype(dtype)
        dx = rk.ROCArray(x)
        for f, op in (("identity", "add_sum"), ("abs2", "max"), ("identity", "min")):
            got = rk.Array(rk.mapreduce(f, op, dx, dims=dims))
            want = orc.mapreduce(f, op, x, dims=dims)
            if np.dtype(dtype).kind == "f" and op == "add_sum":
                np.testing.assert_allclose(got, want, rtol=1e-5 if dtype == np.float32 else 1e-12, atol=1e-2)
            else:
                assert np.array_equal(got, want.astype(got.dtype))
    if isinstance(dims, int):
        _check_findminmax(rk, orc, rng.integers(-4, 5, shape).astype(np.float32), dims)
        _check_findminmax(rk, orc, rng.standard_normal(shape).astype(np.float64), dims)
    c = rk.count(lambda v: v > 0, rk.ROCArray(x), dims=dims)
    ax = tuple(d - 1 for d in ((dims,) if isinstance(dims, int) else dims))
    assert np.array_equal(rk.Array(c), (x > 0).sum(axis=ax, keepdims=True))


@pytest.mark.parametrize("m", [2, 3, 5, 8, 15, 16, 17, 20, 31, 32, 33, 48, 63, 64, 65, 100, 128, 129, 200, 255, 256])
def test_many_short_contiguous_lines(rk, orc, m):
    """dims=1 with 2 .. 256 elements a line and many lines (sum(A; dims=1) of a 32 x N array): whole lines staged through
    LDS, 1 .. 16 lanes a line.  Line counts that fill a block exactly, leave a ragged last block, and an offset view
    (no 16-byte alignment: the scalar loads)."""
    rng = _rng(83 + m)
    for n in (1024, 4111, 70_001):
        for dtype in (np.float32, np.int64, np.float64, np.uint8):
            x = rng.integers(0 if dtype == np.uint8 else -1000, 200 if dtype == np.uint8 else 1001, (m, n)).astype(dtype)
            dx = rk.ROCArray(x)
            for f, op in (("identity", "add_sum"), ("abs2", "max"), ("identity", "min")):
                if dtype == np.uint8 and f == "abs2":
                    continue
                got = rk.Array(rk.mapreduce(f, op, dx, dims=1))
                want = orc.mapreduce(f, op, x, dims=1)
                if np.dtype(dtype).kind == "f" and op == "add_sum":
                    np.testing.assert_allclose(got, want, rtol=1e-5 if dtype == np.float32 else 1e-12, atol=1e-2)
                else:
                    assert np.array_equal(got, want.astype(got.dtype))
        _check_findminmax(rk, orc, rng.integers(-2, 3, (m, n)).astype(np.float32), 1)        # ties: the first index wins
        _check_findminmax(rk, orc, rng.standard_normal((m, n)), 1)
        c = rk.count(lambda v: v > 0, dx, dims=1)
        assert np.array_equal(rk.Array(c), (x > 0).sum(axis=0, keepdims=True))
    flat = rng.standard_normal(m * 2000 + 3).astype(np.float32)
    v = rk.ROCArray(flat).view_range(4, 3 + m * 2000).reshape(m, 2000)
    got = rk.Array(rk.mapreduce("identity", "add_sum", v, dims=1))
    np.testing.assert_allclose(got, flat[3:3 + m * 2000].reshape(2000, m).sum(axis=1, dtype=np.float64)[None, :], rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("shape,dims", [((2, 8, 5000), 2), ((4, 32, 3001), 2), ((4, 100, 1025), 2), ((16, 20, 2000), 2), ((3, 17, 4099), 2),
                                        ((8, 300, 500), 2), ((32, 32, 1000), 2), ((5, 5, 30_001), 2), ((48, 64, 333), 2), ((63, 65, 129), 2),
                                        ((2, 8, 5, 1000), 2), ((3, 2, 7, 4000), 3), ((2, 2, 2, 2, 9000), (3, 4)), ((7, 2, 100_000), 2)])
def test_short_lines_with_a_narrow_inner_extent(rk, orc, shape, dims):
    """1 < inner < 64 with a short reduced dim and many slabs (sum(A; dims=2) of a 4 x 32 x N array): whole inner x mid
    slabs staged through LDS."""
    rng = _rng(97)
    for dtype in (np.float32, np.int32, np.int64, np.float64, np.uint8):
        x = rng.integers(0 if dtype == np.uint8 else -1000, 200 if dtype == np.uint8 else 1001, shape).astype(dtype)
        dx = rk.ROCArray(x)
        for f, op in (("identity", "add_sum"), ("abs2", "max"), ("identity", "min")):
            if dtype == np.uint8 and f == "abs2":
                continue
            got = rk.Array(rk.mapreduce(f, op, dx, dims=dims))
            want = orc.mapreduce(f, op, x, dims=dims)
            if np.dtype(dtype).kind == "f" and op == "add_sum":
                np.testing.assert_allclose(got, want, rtol=1e-5 if dtype == np.float32 else 1e-12, atol=1e-2)
            else:
                assert np.array_equal(got, want.astype(got.dtype))
    if isinstance(dims, int):
        _check_findminmax(rk, orc, rng.integers(-2, 3, shape).astype(np.float32), dims)
        _check_findminmax(rk, orc, rng.standard_normal(shape), dims)
    c = rk.count(lambda v: v > 100, dx, dims=dims)
    ax = tuple(d - 1 for d in ((dims,) if isinstance(dims, int) else dims))
    assert np.array_equal(rk.Array(c), (x > 100).sum(axis=ax, keepdims=True))


@pytest.mark.parametrize("shape,dims", [((4, 20_000, 4), (1, 3)), ((64, 16, 64), (1, 3)), ((8, 300, 8), (1, 3)), ((3, 5, 7, 2000), (1, 3)),
                                        ((2, 17_000, 3, 2), (1, 3, 4)), ((100, 3, 100, 5), (1, 3)), ((2, 2, 2, 2, 2, 5000), (1, 3, 5))])
def test_reduced_dims_that_are_no_single_run(rk, orc, shape, dims):
    """Reduced dims separated by kept ones (dims=(1, 3)) in the kernel for arbitrary masks: a lane, a wave or a workgroup
    per output by the number of outputs and of elements each.  findmax / findmin always take it; the reductions take it
    when the intermediate of a two-step fold would not fit the workspace (the last case below)."""
    rng = _rng(131)
    _check_findminmax(rk, orc, rng.integers(-3, 4, shape).astype(np.float32), dims)       # ties: the first index wins
    _check_findminmax(rk, orc, rng.standard_normal(shape), dims)
    _check_findminmax(rk, orc, rng.integers(-1000, 1000, shape).astype(np.int32), dims)
    x = rng.integers(-1000, 1001, shape).astype(np.int64)
    for op in ("add_sum", "max", "min"):
        assert np.array_equal(rk.Array(rk.mapreduce("identity", op, rk.ROCArray(x), dims=dims)), orc.mapreduce("identity", op, x, dims=dims))


def test_two_step_fold_that_does_not_fit(rk, orc):
    x = _rng(137).integers(-1000, 1001, (4, 1_400_000, 4)).astype(np.float32)           # either fold leaves 22 MB
    dx = rk.ROCArray(x)
    assert np.array_equal(rk.Array(rk.maximum(dx, dims=(1, 3))), x.max(axis=(0, 2), keepdims=True))
    np.testing.assert_allclose(rk.Array(rk.sum(dx, dims=(1, 3))), x.sum(axis=(0, 2), keepdims=True, dtype=np.float64), rtol=1e-5, atol=1e-2)


@pytest.mark.parametrize("dtype,utype", [(np.float32, np.uint32), (np.float64, np.uint64), (np.float16, np.uint16)])
def test_findmax_findmin_return_the_nan_itself(rk, dtype, utype):
    # Julia returns the winning ELEMENT: a negative NaN or one with a payload comes back bit for bit (the first NaN wins)
    bits = {np.float32: (0xffc00001, 0x7fc12345, 0x7f800001), np.float64: (0xfff8000000000001, 0x7ff8000000abcdef, 0x7ff0000000000001),
            np.float16: (0xfe01, 0x7e55, 0x7c01)}[dtype]
    rng = _rng(77)
    for shape, dims in (((5000,), None), ((300, 40), 1), ((300, 40), 2), ((6, 70000), 1)):
        h = rng.standard_normal(shape).astype(dtype)
        u = h.view(utype).reshape(-1)
        pos = rng.choice(u.size, 3, replace=False)
        for p_, b in zip(pos, bits):
            u[p_] = b
        d = rk.ROCArray(h)
        for fn in (rk.findmax, rk.findmin):
            if dims is None:
                v, i = fn(d)
                first = int(np.flatnonzero(np.isnan(h.reshape(-1)))[0])
                assert int(i) == first + 1
                assert np.array(v, dtype=dtype).view(utype) == h.reshape(-1).view(utype)[first]
            else:
                v, i = fn(d, dims=dims)
                gv = rk.Array(v)
                gi = np.moveaxis(rk.Array(i), 0, -1).reshape(-1, 2) - 1
                picked = h[gi[:, 0], gi[:, 1]]
                assert np.array_equal(gv.reshape(-1).view(utype), picked.view(utype))       # value == A[index], bit for bit
                ax = dims - 1
                has_nan = np.isnan(h).any(axis=ax)
                first_nan = np.argmax(np.isnan(h), axis=ax)
                assert np.array_equal(gi[:, ax][has_nan.reshape(-1)], first_nan.reshape(-1)[has_nan.reshape(-1)])


@pytest.mark.parametrize("dtype", [np.bool_, np.uint8, np.float16, np.int8, np.int16, np.uint16])
@pytest.mark.parametrize("shape", [(1024, 40), (2048, 300), (512, 7, 3), (4096, 129)])
def test_narrow_elements_along_rows(rk, orc, dtype, shape):
    """sum / maximum over dims=2 of 1- and 2-byte elements with long contiguous rows: a strip of the strided kernel is
    64 sixteen-byte vectors = 512 or 1024 columns wide, more than a workgroup has threads (an earlier version folded
    and stored only the first 256 columns of every strip)."""
    rng = np.random.default_rng(77)
    if np.dtype(dtype) == np.bool_:
        x = rng.random(shape) < 0.3
    elif np.dtype(dtype).kind == "f":
        x = rng.standard_normal(shape).astype(dtype)
    else:
        info = np.iinfo(dtype)
        x = rng.integers(info.min, info.max + 1, shape).astype(dtype)
    dx = rk.ROCArray(x)
    for op in (("add_sum",) if np.dtype(dtype) == np.bool_ else ("add_sum", "max")):      # count(A; dims=2) for Bool
        got = rk.Array(rk.mapreduce("identity", op, dx, dims=2))
        want = orc.mapreduce("identity", op, x, dims=2)
        assert got.dtype == orc.reduce_eltype(op, x.dtype) and got.shape == want.shape
        if got.dtype.kind == "f":
            np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=2e-3, atol=2e-3)
        else:
            assert np.array_equal(got, want.astype(got.dtype))
    if np.dtype(dtype) != np.bool_:
        gv, gi = rk.findmax(dx, dims=2)
        ov, oi = orc.findmax(x, dims=2)
        assert np.array_equal(rk.Array(gv), ov) and np.array_equal(np.moveaxis(rk.Array(gi), 0, -1), oi)


@pytest.mark.parametrize("m", [257, 300, 400, 511, 512])
def test_lines_of_a_few_hundred_elements(rk, orc, m):
    """dims=1 with lines of 257 .. 512 elements: whole lines through LDS, 16 lanes a line (a wave a line idles most of
    its second round: 300 elements 59 us -> 47 us for 2^26 bytes)."""
    rng = np.random.default_rng(m)
    for dtype in (np.float32, np.int32, np.float64):
        x = (rng.standard_normal((m, 3001)) * 100).astype(dtype)
        dx = rk.ROCArray(x)
        got = rk.Array(rk.mapreduce("identity", "add_sum", dx, dims=1))
        want = orc.mapreduce("identity", "add_sum", x, dims=1)
        if np.dtype(dtype).kind == "f":
            np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-3 if dtype == np.float32 else 1e-9)
        else:
            assert np.array_equal(got, want)
        assert np.array_equal(rk.Array(rk.mapreduce("abs", "max", dx, dims=1)), orc.mapreduce("abs", "max", x, dims=1).astype(dtype))
        gv, gi = rk.findmax(dx, dims=1)
        ov, oi = orc.findmax(x, dims=1)
        assert np.array_equal(rk.Array(gv), ov) and np.array_equal(np.moveaxis(rk.Array(gi), 0, -1), oi)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(64, 8192), (32, 12288), (3, 40960), (100, 6000, 3), (48, 4099), (24, 4096 * 5, 2),
                                   (130, 8192), (7, 8192)])
def test_long_reduced_dim_behind_a_short_contiguous_one(rk, orc, shape):
    """dims=2 of a (short, long[, outer]) array: f consecutive rows are reduced as one row of f * short elements into a
    temporary that a second reduction folds (64 x 1_000_000 Float32: 90 -> 53 us).  4099 rows have no usable factor and
    take the plain strided kernel; 7 x 8192 needs a factor that makes the row a whole number of 16-byte vectors."""
    rng = np.random.default_rng(sum(shape))
    for dtype in (np.float32, np.int32, np.float16, np.uint8, np.float64):
        x = (rng.integers(-50, 50, size=shape) if np.dtype(dtype).kind != "f" else rng.standard_normal(shape) * 4).astype(dtype)
        dx = rk.ROCArray(x)
        got = rk.Array(rk.mapreduce("identity", "add_sum", dx, dims=2))
        want = orc.mapreduce("identity", "add_sum", x, dims=2)
        if np.dtype(dtype).kind == "f":
            tol = {np.float16: (2e-2, 0.5), np.float32: (1e-5, 1e-3), np.float64: (1e-12, 1e-10)}[dtype]
            np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=tol[0], atol=tol[1])
        else:
            assert got.dtype == want.dtype and np.array_equal(got, want)
        assert np.array_equal(rk.Array(rk.mapreduce("identity", "max", dx, dims=2)), orc.mapreduce("identity", "max", x, dims=2))
        if dtype in (np.float32, np.int32):
            init = np.asarray(3, dtype=want.dtype)
            g2 = rk.Array(rk.mapreduce("abs2", "add_sum", dx, dims=2, init=init[()]))
            w2 = orc.mapreduce("abs2", "add_sum", x, dims=2, init=init[()])
            if dtype == np.float32:
                np.testing.assert_allclose(g2, w2, rtol=1e-5, atol=1e-2)
            else:
                assert np.array_equal(g2, w2)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(200, 3, 50), (70, 16, 60), (1001, 5, 7), (65, 2, 100), (4099, 9, 2), (33, 200, 40), (7, 100, 300), (63, 70, 9)])
def test_short_or_medium_reduced_dim_in_the_middle(rk, orc, shape):
    """dims=2 of a 3-d array.  A reduced extent <= 16 behind >= 64 contiguous columns: a lane per group of four (two)
    columns, 16-byte loads at element-aligned addresses, the last group of a row starting early (1001, 65, 4099 columns).
    64 .. 1023 rows behind fewer than 64 columns, in slabs above 16 KiB: runs of whole rows, not a wave per line."""
    rng = np.random.default_rng(sum(shape))
    for dtype in (np.float32, np.int32, np.float64, np.int64):
        x = (rng.standard_normal(shape) * 100).astype(dtype)
        dx = rk.ROCArray(x)
        got = rk.Array(rk.mapreduce("identity", "add_sum", dx, dims=2))
        want = orc.mapreduce("identity", "add_sum", x, dims=2)
        if np.dtype(dtype).kind == "f":
            np.testing.assert_allclose(got, want, rtol=1e-5 if dtype == np.float32 else 1e-12, atol=1e-2 if dtype == np.float32 else 1e-9)
        else:
            assert got.dtype == want.dtype and np.array_equal(got, want)
        assert np.array_equal(rk.Array(rk.mapreduce("abs", "max", dx, dims=2)), orc.mapreduce("abs", "max", x, dims=2))
        gv, gi = rk.findmin(dx, dims=2)
        ov, oi = orc.findmin(x, dims=2)
        assert np.array_equal(rk.Array(gv), ov) and np.array_equal(np.moveaxis(rk.Array(gi), 0, -1), oi)
