"""GPU parity of accumulate / cumsum / cumprod / findall against the oracle, through the C ABI.

Tolerances: integer scans bit-exact (wraparound); Float32 scans rtol 1e-4 against a Float64 host scan
(atol covers prefixes that pass near zero)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL = 1e-4


def _rng(seed):
    return np.random.default_rng(seed)


SIZES = [0, 1, 2, 3, 10, 63, 64, 65, 1000, 4095, 4096, 4097, 8192, 10_000, 16384, 16385, 100_003, (1 << 20) + 5]


@pytest.mark.parametrize("n", SIZES)
def test_accumulate_f64_sizes(rk, orc, n):
    # test/core/rocarray_base.jl:194-201 (Float64, with and without init)
    x = _rng(n).random(n)
    d = rk.ROCArray(x)
    np.testing.assert_allclose(rk.Array(rk.accumulate("add", d)), orc.accumulate("add", x), rtol=1e-12)
    init = 0.37
    np.testing.assert_allclose(rk.Array(rk.accumulate("add", d, init=init)), orc.accumulate("add", x, init=init), rtol=1e-12)


@pytest.mark.parametrize("n", SIZES)
def test_cumsum_i32_exact(rk, orc, n):
    x = _rng(n + 1).integers(-1000, 1001, n, dtype=np.int32)
    got = rk.cumsum(rk.ROCArray(x))
    assert got.dtype == np.int32
    assert np.array_equal(rk.Array(got), orc.cumsum(x))


def test_cumsum_i32_wraps(rk, orc):
    x = np.full(100_000, 2_000_000_000, dtype=np.int32)
    want = np.cumsum(x.astype(np.int64)).astype(np.uint64).astype(np.uint32).view(np.int32)   # mod 2^32
    assert np.array_equal(orc.cumsum(x), want)
    assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(x))), want)


@pytest.mark.parametrize("n", [1, 100, 4096, 4097, 50_000, (1 << 19) + 1])
def test_cumsum_f32(rk, orc, n):
    x = _rng(n).random(n, dtype=np.float32)
    want = orc.cumsum(x)
    np.testing.assert_allclose(rk.Array(rk.cumsum(rk.ROCArray(x))), want, rtol=RTOL)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
@pytest.mark.parametrize("op", ["add", "mul", "max", "min"])
@pytest.mark.parametrize("inclusive", [True, False])
def test_ops_dtypes_exclusive(rk, orc, dtype, op, inclusive):
    rng = _rng(21)
    n = 20_000
    if op == "mul":
        x = (rng.random(n) * 0.002 + 0.999).astype(dtype) if np.dtype(dtype).kind == "f" else rng.integers(-2, 3, n).astype(dtype)
        init = 2
    else:
        x = (rng.standard_normal(n) * 50).astype(dtype)
        init = 3
    got = rk.Array(rk.accumulate(op, rk.ROCArray(x), init=init, inclusive=inclusive))
    want = orc.accumulate(op, x, init=init, inclusive=inclusive)
    if np.dtype(dtype).kind == "f" and op in ("add", "mul"):
        np.testing.assert_allclose(got, want, rtol=RTOL if dtype == np.float32 else 1e-11, atol=2e-2 if (op == "add" and dtype == np.float32) else 1e-9)
    else:
        assert np.array_equal(got, want.astype(dtype))


DIM_CASES = [
    ((2,), 2), ((3, 4, 5), 2), ((1, 70, 50, 20), 3),            # test/core/rocarray_base.jl:204-213
    ((3, 4, 5), 1), ((3, 4, 5), 3), ((64, 64), 1), ((64, 64), 2), ((100, 1000), 1), ((100, 1000), 2),
    ((512, 1000), 1), ((512, 1000), 2), ((3, 100_000), 1), ((3, 100_000), 2), ((100_000, 3), 1), ((100_000, 3), 2),
    ((4096, 33), 1), ((4100, 33), 1), ((9000, 7), 1), ((257, 129, 5), 2), ((256, 40, 3), 2), ((40, 50), 3),
    ((1024, 300), 1), ((1000, 300), 1), ((300, 70), 1), ((20, 5000), 1),
]


@pytest.mark.parametrize("shape,dims", DIM_CASES)
def test_accumulate_dims_i64_exact(rk, orc, shape, dims):
    x = _rng(22).integers(-10**12, 10**12, shape, dtype=np.int64)
    assert np.array_equal(rk.Array(rk.accumulate("add", rk.ROCArray(x), dims=dims)), orc.accumulate("add", x, dims=dims))


@pytest.mark.parametrize("shape,dims", DIM_CASES)
def test_cumsum_dims_f32(rk, orc, shape, dims):
    x = _rng(23).random(shape, dtype=np.float32)
    np.testing.assert_allclose(rk.Array(rk.cumsum(rk.ROCArray(x), dims=dims)), orc.cumsum(x, dims=dims), rtol=RTOL)


@pytest.mark.parametrize("shape,dims", [((3, 4, 5), 2), ((4096, 9), 1), ((9000, 3), 1), ((130, 70), 2)])
def test_exclusive_with_init_dims(rk, orc, shape, dims):
    x = _rng(24).integers(-100, 100, shape, dtype=np.int32)
    got = rk.Array(rk.accumulate("add", rk.ROCArray(x), dims=dims, init=7, inclusive=False))
    assert np.array_equal(got, orc.accumulate("add", x, dims=dims, init=7, inclusive=False))


SLICED_CASES = [((128, 4096), 2), ((100, 5001), 2), ((67, 3000, 2), 2), ((256, 1 << 14), 2), ((64, 200, 3), 2), ((1000, 777), 2),
                ((8, 16, 2500), 3)]


@pytest.mark.parametrize("shape,dims", SLICED_CASES)
@pytest.mark.parametrize("op,inclusive", [("add", True), ("add", False), ("max", True), ("min", False)])
def test_long_scans_across_rows(rk, orc, shape, dims, op, inclusive):
    # few columns, many rows: the rows are cut into slices that scan independently from carried-in prefixes
    x = _rng(31).integers(-10**6, 10**6, shape, dtype=np.int32)
    got = rk.Array(rk.accumulate(op, rk.ROCArray(x), dims=dims, init=-5, inclusive=inclusive))
    assert np.array_equal(got, orc.accumulate(op, x, dims=dims, init=-5, inclusive=inclusive))


@pytest.mark.parametrize("dtype", [np.float64, np.int64, np.bool_])
def test_long_scans_across_rows_dtypes(rk, orc, dtype):
    rng = _rng(32)
    x = (rng.random((192, 5000)) < 0.3) if dtype == np.bool_ else (rng.standard_normal((192, 5000)) * 100).astype(dtype)
    d = rk.ROCArray(x)
    got = rk.Array(rk.cumsum(d, dims=2))
    want = orc.cumsum(x, dims=2)
    if dtype == np.float64:
        np.testing.assert_allclose(got, want, rtol=1e-11, atol=1e-9)
    else:
        assert np.array_equal(got, want)
    if dtype != np.bool_:
        rk.accumulate_("add", d, d, dims=2)                         # in place
        assert np.array_equal(rk.Array(d), got)


def test_in_place(rk, orc):
    # test/core/rocarray_base.jl:216-220
    x = _rng(25).random(2)
    d = rk.ROCArray(x)
    out = rk.accumulate_("add", d, d)
    assert out is d
    np.testing.assert_allclose(rk.Array(d), np.cumsum(x))
    y = _rng(26).integers(-1000, 1000, 1 << 18, dtype=np.int32)
    dy = rk.ROCArray(y)
    rk.accumulate_("add", dy, dy)
    assert np.array_equal(rk.Array(dy), orc.cumsum(y))


def test_cumprod_and_doctest(rk, orc):
    assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(np.array([1, 2, 3, 4])))), [1, 3, 6, 10])   # arrays.md:91-96
    x = _rng(27).random(2)
    np.testing.assert_allclose(rk.Array(rk.cumprod(rk.ROCArray(x))), np.cumprod(x))


def test_unaligned_view_scan(rk, orc):
    x = _rng(28).integers(-1000, 1000, 50_001, dtype=np.int32)
    d = rk.ROCArray(x)
    v = d.view_range(2, 50_001)
    assert np.array_equal(rk.Array(rk.cumsum(v)), orc.cumsum(x[1:]))


def test_repeated_scans_bump_generation(rk, orc):
    # many look-back scans in a row through one workspace: stale descriptors must never be accepted
    rng = _rng(29)
    for it in range(12):
        n = int(rng.integers(5000, 300_000))
        x = rng.integers(-1000, 1001, n, dtype=np.int32)
        assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(x))), orc.cumsum(x)), (it, n)


def test_config3_full_size(rk, orc):
    x = orc.config_inputs("cumsum_i32")["x"]                      # 2^27 Int32
    got = rk.Array(rk.cumsum(rk.ROCArray(x)))
    assert np.array_equal(got, np.cumsum(x, dtype=np.int32))
    del got
    B = orc.config_inputs("cumsum_f32_dims1")["B"]                # 4096 x 16384 Float32
    got = rk.Array(rk.cumsum(rk.ROCArray(B), dims=1))
    np.testing.assert_allclose(got, np.cumsum(B.astype(np.float64), axis=0), rtol=RTOL)


def test_bool_scan_and_findall(rk, orc):
    b = _rng(30).random(100_000) < 0.25
    got = rk.cumsum(rk.ROCArray(b))
    assert got.dtype == np.int64
    assert np.array_equal(rk.Array(got), np.cumsum(b))
    assert np.array_equal(rk.Array(rk.findall(rk.ROCArray(b))), orc.findall(b))
    # test/hip_rocarray/indexing.jl:5-18 shapes
    for shape in [(16,), (1, 16), (3, 1, 16), (33, 65)]:
        m = _rng(31).random(shape) < 0.5
        got = rk.Array(rk.findall(rk.ROCArray(m)))
        want = orc.findall(m)
        assert np.array_equal(got if m.ndim == 1 else got.T, want)
    assert len(rk.findall(rk.ROCArray(np.zeros(100, dtype=bool)))) == 0


@pytest.mark.parametrize("dtype", [np.uint32, np.uint64])
def test_unsigned_scans_wrap(rk, orc, dtype):
    rng = _rng(33)
    info = np.iinfo(dtype)
    for shape, dims in [((300_001,), 1), ((300, 70), 1), ((300, 70), 2), ((64, 3000), 2)]:
        x = rng.integers(0, info.max, shape, dtype=dtype, endpoint=True)
        got = rk.accumulate("add", rk.ROCArray(x), dims=dims)
        assert got.dtype == dtype
        with np.errstate(over="ignore"):
            assert np.array_equal(rk.Array(got), np.cumsum(x, axis=dims - 1, dtype=dtype))
        assert np.array_equal(rk.Array(rk.accumulate("max", rk.ROCArray(x), dims=dims)), np.maximum.accumulate(x, axis=dims - 1))


NARROW_CASES = [((3, 1_000_000), 2), ((2, 70_001), 2), ((5, 9000, 3), 2), ((17, 33_333), 2), ((63, 20_000), 2), ((7, 3, 40_000), 3),
                ((3, 5, 9001, 2), 3), ((63, 65), 2), ((2, 2_100_000), 2)]


@pytest.mark.parametrize("shape,dims", NARROW_CASES)
def test_narrow_inner_long_lines(rk, orc, shape, dims):
    # accumulate(+, 3 x 1_000_000; dims=2) of perf/array.jl:77,84: few columns, very long lines
    rng = _rng(34)
    x = rng.integers(-1000, 1000, shape, dtype=np.int32)
    d = rk.ROCArray(x)
    assert np.array_equal(rk.Array(rk.accumulate("add", d, dims=dims)), orc.accumulate("add", x, dims=dims))
    assert np.array_equal(rk.Array(rk.accumulate("max", d, dims=dims, init=5, inclusive=False)),
                          orc.accumulate("max", x, dims=dims, init=5, inclusive=False))
    xf = rng.random(shape)
    np.testing.assert_allclose(rk.Array(rk.cumsum(rk.ROCArray(xf), dims=dims)), orc.cumsum(xf, dims=dims), rtol=1e-11)
    b = rng.random(shape) < 0.5
    assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(b), dims=dims)), orc.cumsum(b, dims=dims))       # Bool -> Int64
    rk.accumulate_("add", d, d, dims=dims)                                                             # in place
    assert np.array_equal(rk.Array(d), orc.accumulate("add", x, dims=dims))


@pytest.mark.parametrize("shape", [(16, 100_000), (4, 50_001), (8, 3, 7000), (12, 1000), (2, 100_000), (16, 1), (6, 999), (20, 3001), (128, 500), (100, 777), (64, 1000), (36, 5, 41)])
def test_short_contiguous_lines(rk, orc, shape):
    rng = _rng(35)
    for dtype in (np.float32, np.float64, np.int32, np.int64):
        x = (rng.standard_normal(shape) * 100).astype(dtype)
        got = rk.Array(rk.accumulate("add", rk.ROCArray(x), dims=1, init=3, inclusive=False))
        want = orc.accumulate("add", x, dims=1, init=3, inclusive=False)
        if np.dtype(dtype).kind == "f":
            np.testing.assert_allclose(got, want, rtol=RTOL if dtype == np.float32 else 1e-12, atol=1e-3 if dtype == np.float32 else 1e-9)
        else:
            assert np.array_equal(got, want)
        assert np.array_equal(rk.Array(rk.accumulate("max", rk.ROCArray(x), dims=1)), orc.accumulate("max", x, dims=1))
    b = rng.random(shape) < 0.5
    assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(b), dims=1)), orc.cumsum(b, dims=1))


@pytest.mark.parametrize("m", [3, 5, 6, 7, 9, 13, 15, 17, 18, 31, 33, 63, 65, 101, 127, 129, 130, 255, 256])
def test_short_contiguous_lines_of_any_length(rk, orc, m):
    """dims=1 with lines of 3 .. 256 elements that are no whole number of 16-byte vectors (cumsum of a 15 x N array):
    whole lines staged through LDS, 1 .. 16 lanes a line; exact and ragged last blocks, inclusive and exclusive, an
    unaligned view, a Bool source."""
    rng = _rng(91 + m)
    for n in (1024, 4111, 30_001):
        for dtype in (np.float32, np.float64, np.int32, np.int64):
            x = rng.integers(-100, 101, (m, n)).astype(dtype)
            dx = rk.ROCArray(x)
            for op, init, inclusive in (("add", None, True), ("add", 3, False), ("max", None, True), ("min", -5, True)):
                got = rk.Array(rk.accumulate(op, dx, dims=1, init=init, inclusive=inclusive))
                want = orc.accumulate(op, x, dims=1, init=init, inclusive=inclusive)
                assert np.array_equal(got, want.astype(got.dtype))          # small integers: Float32 sums are exact too
        xf = rng.standard_normal((m, n)).astype(np.float32)
        got = rk.Array(rk.cumsum(rk.ROCArray(xf), dims=1))
        np.testing.assert_allclose(got, orc.cumsum(xf, dims=1), rtol=RTOL, atol=1e-4)
        b = rng.random((m, n)) < 0.5
        assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(b), dims=1)), orc.cumsum(b, dims=1))
    flat = rng.integers(-50, 51, m * 1500 + 3).astype(np.float32)
    v = rk.ROCArray(flat).view_range(4, 3 + m * 1500).reshape(m, 1500)
    got = rk.Array(rk.cumsum(v, dims=1))
    assert np.array_equal(got, np.cumsum(flat[3:3 + m * 1500].reshape(1500, m), axis=1).T)


@pytest.mark.parametrize("shape,dims", [((2, 8, 5000), 2), ((4, 32, 3001), 2), ((4, 100, 1025), 2), ((16, 20, 2000), 2), ((3, 17, 4099), 2),
                                        ((8, 300, 500), 2), ((32, 32, 1000), 2), ((5, 5, 30_001), 2), ((48, 64, 333), 2), ((63, 65, 129), 2),
                                        ((2, 8, 5, 1000), 2), ((3, 2, 7, 4000), 3), ((64, 16, 300), 2), ((100, 7, 1000), 2), ((7, 2, 100_000), 2), ((2, 1000, 600), 2), ((3, 333, 400), 2), ((1, 4001, 1), 2)])
def test_short_lines_with_a_narrow_inner_extent(rk, orc, shape, dims):
    """A short scanned dim behind a narrow inner extent, many slabs (cumsum(A; dims=2) of a 4 x 32 x N array): whole
    inner x mid slabs staged through LDS."""
    rng = _rng(101)
    for dtype in (np.float32, np.float64, np.int32, np.int64):
        x = rng.integers(-100, 101, shape).astype(dtype)
        dx = rk.ROCArray(x)
        for op, init, inclusive in (("add", None, True), ("add", 3, False), ("max", None, True), ("min", -5, True)):
            got = rk.Array(rk.accumulate(op, dx, dims=dims, init=init, inclusive=inclusive))
            want = orc.accumulate(op, x, dims=dims, init=init, inclusive=inclusive)
            assert np.array_equal(got, want.astype(got.dtype))              # small integers: Float32 sums are exact too
    xf = rng.standard_normal(shape).astype(np.float32)
    np.testing.assert_allclose(rk.Array(rk.cumsum(rk.ROCArray(xf), dims=dims)), orc.cumsum(xf, dims=dims), rtol=RTOL, atol=1e-4)
    b = rng.random(shape) < 0.5
    assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(b), dims=dims)), orc.cumsum(b, dims=dims))


@pytest.mark.parametrize("dtype", [np.int8, np.uint8, np.int16, np.uint16, np.float16])
def test_narrow_element_types(rk, orc, dtype):
    """accumulate / cumsum / cumprod of 1- and 2-byte elements, native in rk_accumulate: read narrow, scanned in the next
    wider type, stored narrow -- one kernel, through every kernel family (shapes below).  Integers wrap in their own
    type, bit-exact; Float16 within a few Float16 roundings of the Float64 scan (AcceleratedKernels rounds after every
    step, the native path once)."""
    rng = np.random.default_rng(91)
    dt = np.dtype(dtype)
    shapes = (((1000,), 1), ((70_001,), 1), ((300, 70), 1), ((300, 70), 2), ((5, 64, 9), 2), ((200_000,), None),
              (((1 << 22) + 40,), 1),          # long line: single pass with look-back
              ((4096, 700), 1),                # a tile a line
              ((16, 40_000), 1), ((15, 40_001), 1),   # short lines: lane groups / whole slabs through LDS
              ((1024, 2048), 2), ((257, 3000), 2),    # across rows: single pass / strips
              ((3, 200_000), 2), ((64, 30_000), 2),   # narrow inner extent, long lines
              ((4, 32, 5000), 2), ((300, 3, 200), 2)) # short scanned dim behind a narrow / a long inner extent
    for shape, dims in shapes:
        if dt.kind == "f":
            x = (rng.random(shape) * 0.01).astype(dt)
        else:
            info = np.iinfo(dt)
            x = rng.integers(info.min, info.max + 1, shape).astype(dt)
        dx = rk.ROCArray(x)
        for op in ("add", "max", "min", "mul"):
            if op == "mul":
                # Float16: factors 2, 1/2, 2, ... along the scanned dim keep every running product within 1 .. 2
                x2 = (rng.integers(1, 3, shape).astype(dt) if dt.kind != "f"
                      else np.where(np.indices(shape)[(dims or 1) - 1] % 2 == 0, 2.0, 0.5).astype(dt))
                src, dsrc = x2, rk.ROCArray(x2)
            else:
                src, dsrc = x, dx
            got = rk.Array(rk.accumulate(op, dsrc, dims=dims))
            want = orc.accumulate(op, src, dims=dims)
            assert got.dtype == dt and got.shape == src.shape
            if dt.kind == "f":
                np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=4e-3, atol=1e-4)
            else:
                assert np.array_equal(got, want.astype(dt))
        # exclusive with init, and in place
        init = dt.type(3)
        got = rk.Array(rk.accumulate("add", dx, dims=dims, init=init, inclusive=False))
        want = orc.accumulate("add", x, dims=dims, init=init, inclusive=False)
        if dt.kind == "f":
            np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=4e-3, atol=1e-4)
        else:
            assert np.array_equal(got, want.astype(dt))
        dy = rk.ROCArray(x)
        assert rk.accumulate_("add", dy, dy, dims=dims) is dy
        want = orc.accumulate("add", x, dims=dims)
        if dt.kind == "f":
            np.testing.assert_allclose(rk.Array(dy).astype(np.float64), want.astype(np.float64), rtol=4e-3, atol=1e-4)
        else:
            assert np.array_equal(rk.Array(dy), want.astype(dt))


@pytest.mark.parametrize("dtype", [np.int8, np.uint8, np.int16, np.uint16])
def test_long_lines_of_narrow_integers(rk, orc, dtype):
    """Lines of 1- and 2-byte integers long enough for the packed tiles of the single-pass scan (128 KiB of elements a
    tile, kept packed in the registers): every operator, inclusive and exclusive with an init, a last tile that is
    nearly empty or nearly full, several lines, in place.  The same arrays through the widened tiles (a length that is
    no whole number of 16-byte vectors) as a cross-check of the shapes.  Bit-exact against the oracle."""
    rng = np.random.default_rng(94)
    dt = np.dtype(dtype)
    info = np.iinfo(dt)
    tile = 16 * 64 * 8 * (16 // dt.itemsize)
    shapes = (((12 * tile + 48,), 1), ((13 * tile - 16,), 1), ((11 * tile, 3), 1), ((12 * tile + 3,), 1))
    for shape, dims in shapes:
        x = rng.integers(info.min, info.max + 1, shape).astype(dt)
        dx = rk.ROCArray(x)
        for op in ("add", "mul", "max", "min", "and", "or", "xor"):
            src, d = x, dx
            if op == "mul":
                src = rng.integers(1, 4, shape).astype(dt)
                d = rk.ROCArray(src)
            elif op in ("max", "min"):
                # a slowly drifting sequence, so that the running extremum keeps changing along the line
                src = (np.arange(x.size).reshape(shape, order="F") // 7000 * (1 if op == "max" else -1) + rng.integers(-3, 4, shape)).astype(dt)
                d = rk.ROCArray(src)
            got = rk.Array(rk.accumulate(op, d, dims=dims))
            assert got.dtype == dt and np.array_equal(got, orc.accumulate(op, src, dims=dims).astype(dt)), (shape, op)
            init = dt.type(src.reshape(-1)[5])
            got = rk.Array(rk.accumulate(op, d, dims=dims, init=init, inclusive=False))
            assert np.array_equal(got, orc.accumulate(op, src, dims=dims, init=init, inclusive=False).astype(dt)), (shape, op, "exclusive")
        if info.min < 0:
            # an init below every element: the exclusive scan's first value is the init itself
            init = dt.type(info.min)
            got = rk.Array(rk.accumulate("max", dx, dims=dims, init=init, inclusive=False))
            assert np.array_equal(got, orc.accumulate("max", x, dims=dims, init=init, inclusive=False).astype(dt))
        dy = rk.ROCArray(x)
        assert rk.accumulate_("add", dy, dy, dims=dims) is dy
        assert np.array_equal(rk.Array(dy), orc.accumulate("add", x, dims=dims).astype(dt))


@pytest.mark.parametrize("m", [8, 9, 11, 129, 255, 1001, 2047, 2049, 3001, 4095, 4097, 8189, 8190, 8191])
def test_lines_that_start_at_odd_addresses(rk, orc, m):
    """cumsum(A; dims=1) with a line length that is no whole number of 16-byte vectors: every line starts at another
    alignment; the kernels take 16 bytes a lane at element-aligned addresses and only the vector that the line's end cuts
    element by element.  A workgroup per line, a wave per line, and (8190 / 8191 Float32 upwards) the chained tiles.
    Integers bit-exact, floats rtol 1e-4 of the Float64 scan."""
    rng = np.random.default_rng(m)
    # fewer than 64 lines: a workgroup per line; 130 lines of up to 1024 elements: a wave per line
    for dtype, n in ((np.float32, 37), (np.int32, 5), (np.float64, 6), (np.int64, 1), (np.float32, 130), (np.int64, 67)):
        if (dtype in (np.float64, np.int64) and m > 4097) or (n > 64 and m > 1024):
            continue
        x = (rng.standard_normal((m, n)) * 10).astype(dtype)
        dx = rk.ROCArray(x)
        for op, inclusive, init in (("add", True, None), ("max", True, None), ("add", False, dtype(7)), ("min", True, dtype(-2))):
            got = rk.Array(rk.accumulate(op, dx, dims=1, init=init, inclusive=inclusive))
            want = orc.accumulate(op, x, dims=1, init=init, inclusive=inclusive)
            if np.dtype(dtype).kind == "f" and op == "add":
                np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-3 if dtype == np.float32 else 1e-9)
            else:
                assert np.array_equal(got, want.astype(dtype)), (dtype, op)
    b = rng.random((m, 9)) < 0.3                                   # Bool -> Int64: one-byte input vectors
    assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(b), dims=1)), orc.accumulate("add", b, dims=1))
    # a view whose first element sits at an odd address, one line and many
    flat = (rng.standard_normal(m * 3 + 5) * 10).astype(np.float32)
    d = rk.ROCArray(flat)
    v = d.view_range(4, m + 3)                                     # elements 4 .. m + 3 (1-based): byte offset 12
    np.testing.assert_allclose(rk.Array(rk.cumsum(v)), np.cumsum(flat[3:m + 3].astype(np.float64)), rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.float64, np.int64])
def test_long_lines_at_odd_addresses(rk, orc, dtype):
    """Lines longer than a tile that start at element-aligned but not 16-byte-aligned addresses -- a view x[2:end], the
    columns of a 20001 x N matrix -- take the single-pass kernel with its 16-byte accesses at element-aligned addresses:
    one long line (many tiles, the last one partly filled), several lines of a few tiles each, in place, exclusive with
    an init.  Integers bit-exact, floats rtol 1e-4 of the Float64 scan."""
    rng = np.random.default_rng(77)
    dt = np.dtype(dtype)

    def check(got, x, dims, **kw):
        want = orc.accumulate("add", x, dims=dims, **kw)
        if dt.kind == "f":
            np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-2 if dt == np.float32 else 1e-8)
        else:
            assert np.array_equal(got, want.astype(dt))

    n = (1 << 22) + 37
    flat = rng.integers(-100, 101, n + 8).astype(dt)
    d = rk.ROCArray(flat)
    for first in (2, 4):                                           # byte offsets 1 and 3 elements
        v = d.view_range(first, first + n - 1)
        x = flat[first - 1:first - 1 + n]
        check(rk.Array(rk.cumsum(v)), x, 1)
        check(rk.Array(rk.accumulate("add", v, init=dt.type(5), inclusive=False)), x, 1, init=dt.type(5), inclusive=False)
        if dt.kind != "f":
            assert np.array_equal(rk.Array(rk.accumulate("max", v)), orc.accumulate("max", x, dims=1))
    for shape in ((20_001, 150), (70_003, 31), (300_001, 6)):
        x = rng.integers(-100, 101, shape).astype(dt)
        check(rk.Array(rk.cumsum(rk.ROCArray(x), dims=1)), x, 1)
        dy = rk.ROCArray(x)
        assert rk.accumulate_("add", dy, dy, dims=1) is dy
        check(rk.Array(dy), x, 1)


@pytest.mark.parametrize("shape", [(257, 300), (1001, 1000), (4097, 130), (65, 5000), (130, 70, 5), (67, 40, 9), (8191, 33),
                                   (200, 3, 50), (1001, 5, 7), (4099, 16, 2), (256, 2, 40)])
def test_scans_across_rows_that_are_no_whole_vectors(rk, orc, shape):
    """cumsum(A; dims=2) with a first extent that is no multiple of the 16-byte vector: every row has another alignment.
    The kernels read and write vectors at element-aligned addresses; the last vector of a row starts four (two)
    elements before the row's end.  All paths: one workgroup per strip, sliced with carried totals, the single pass
    over tiles of rows, and (a scanned extent <= 16) a lane per group of columns.  In place too: there a row's last
    vector would re-read columns another lane has already overwritten, so odd rows take the element-wise kernels."""
    rng = np.random.default_rng(sum(shape))
    for dtype in (np.float32, np.int32, np.float64, np.int64):
        x = (rng.standard_normal(shape) * 10).astype(dtype)
        dx = rk.ROCArray(x)
        for op, inclusive, init in (("add", True, None), ("max", True, None), ("add", False, dtype(3))):
            got = rk.Array(rk.accumulate(op, dx, dims=2, init=init, inclusive=inclusive))
            want = orc.accumulate(op, x, dims=2, init=init, inclusive=inclusive)
            if np.dtype(dtype).kind == "f" and op == "add":
                np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-2 if dtype == np.float32 else 1e-9)
            else:
                assert np.array_equal(got, want.astype(dtype)), (dtype, op)
        rk.accumulate_("add", dx, dx, dims=2)
        want = orc.accumulate("add", x, dims=2)
        if np.dtype(dtype).kind == "f":
            np.testing.assert_allclose(rk.Array(dx), want, rtol=1e-4, atol=1e-2 if dtype == np.float32 else 1e-9)
        else:
            assert np.array_equal(rk.Array(dx), want.astype(dtype))


@pytest.mark.parametrize("shape", [(100, 50_000), (65, 30_011), (128, 9_000), (95, 20_000, 2), (32, 100_001), (33, 40_000, 3), (16, 33_000, 5),
                                   (64, 2_000, 3), (31, 70_000), (128, 4_001), (48, 1921), (17, 200_000)])
def test_short_rows_several_to_a_load(rk, orc, shape):
    """cumsum(A; dims=2) with rows of 128 bytes up to half a strip of columns (32 .. 128 Float32, 16 .. 64 Float64) and long
    lines: a load instruction takes several rows, a group of lanes each, every group scans its consecutive rows in
    registers and one scan across the lanes joins the groups; tiles of rows in launch order with a look-back over the
    column totals.  Odd extents (rows at every alignment, last vector shifted back), several outer indices, partial
    last tiles, and the neighbouring shapes that take the other kernels; in place too."""
    rng = np.random.default_rng(sum(shape))
    for dtype in (np.float32, np.int32, np.float64, np.int64):
        x = (rng.standard_normal(shape) * 10).astype(dtype)
        dx = rk.ROCArray(x)
        for op, inclusive, init in (("add", True, None), ("min", True, None), ("add", False, dtype(3))):
            got = rk.Array(rk.accumulate(op, dx, dims=2, init=init, inclusive=inclusive))
            want = orc.accumulate(op, x, dims=2, init=init, inclusive=inclusive)
            if np.dtype(dtype).kind == "f" and op == "add":
                np.testing.assert_allclose(got, want, rtol=1e-4, atol=5e-2 if dtype == np.float32 else 1e-9)
            else:
                assert np.array_equal(got, want.astype(dtype)), (dtype, op)
        rk.accumulate_("add", dx, dx, dims=2)
        want = orc.accumulate("add", x, dims=2)
        if np.dtype(dtype).kind == "f":
            np.testing.assert_allclose(rk.Array(dx), want, rtol=1e-4, atol=5e-2 if dtype == np.float32 else 1e-9)
        else:
            assert np.array_equal(rk.Array(dx), want.astype(dtype))


@pytest.mark.parametrize("dtype", [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64, np.bool_])
def test_bitwise_scan_operators(rk, orc, dtype):
    """accumulate(&, A), accumulate(|, A), accumulate(xor, A) on integer element types and Bool (what AcceleratedKernels
    accepts through src/kernels/accumulate.jl:1-8 besides + * max min), bit-exact, through every kernel family."""
    rng = np.random.default_rng(93)
    dt = np.dtype(dtype)
    shapes = (((1000,), 1), (((1 << 21) + 40,), 1), ((4096, 300), 1), ((15, 20_001), 1), ((512, 1200), 2), ((3, 100_000), 2),
              ((4, 32, 2000), 2), ((300, 3, 100), 2), ((70_001,), None))
    for shape, dims in shapes:
        if dt == np.bool_:
            x = rng.random(shape) < 0.9
        else:
            # mostly-ones bit patterns, so that & keeps bits alive for a while and | fills up slowly from sparse ones
            x = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, shape, dtype=dt, endpoint=True)
        dx = rk.ROCArray(x)
        for op in ("and", "or", "xor"):
            src = x
            if op == "and" and dt != np.bool_:
                src = x | rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, shape, dtype=dt, endpoint=True)
            elif op == "or" and dt != np.bool_:
                src = x & rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, shape, dtype=dt, endpoint=True) & rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, shape, dtype=dt, endpoint=True)
            d = rk.ROCArray(src) if src is not x else dx
            got = rk.Array(rk.accumulate(op, d, dims=dims))
            assert got.dtype == dt and np.array_equal(got, orc.accumulate(op, src, dims=dims)), (shape, dims, op)
            init = src.reshape(-1)[7]
            got = rk.Array(rk.accumulate(op, d, dims=dims, init=init, inclusive=False))
            assert np.array_equal(got, orc.accumulate(op, src, dims=dims, init=init, inclusive=False)), (shape, dims, op, "exclusive")
    with pytest.raises(NotImplementedError):
        rk.accumulate("xor", rk.ROCArray(np.ones(8, dtype=np.float32)))
