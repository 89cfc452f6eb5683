"""GPU parity of sort / sort! / sortperm / sortperm! (src/kernels/sorting.jl:1-3) against the oracle, through the
C ABI: the sizes and element types of test/hip_rocarray/sorting.jl:5-28 for the default order and rev=true
(values and permutations bit-exact, NaNs compared as equal), plus sizes that span many tiles, special floats,
duplicates (stability) and small-range integers (skipped passes).  The two other forms of that test, `lt=!isless` and
`by=k -> 2k` (:20-26), are native as well: descending order, and map -> sortperm of the keys -> gather."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TYPES = [np.float16, np.float32, np.float64, np.int16, np.int32, np.int64]


def _rand(rng, dtype, n):
    dt = np.dtype(dtype)
    if dt.kind == "f":
        return rng.random(n).astype(dt)                       # rand(T, sz)
    return rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, n, dtype=dt, endpoint=True)


def _check(rk, orc, x):
    xd = rk.ROCArray(x)
    for rev in (False, True):
        want, wperm = orc.sort(x, rev), orc.sortperm(x, rev)
        got = rk.Array(rk.sort(xd, rev=rev))
        assert got.dtype == x.dtype and np.array_equal(got, want, equal_nan=x.dtype.kind == "f"), rev
        if x.dtype.kind == "f":
            assert np.array_equal(np.signbit(got[~np.isnan(got)]), np.signbit(want[~np.isnan(want)]))
        p = rk.Array(rk.sortperm(xd, rev=rev))
        assert p.dtype == np.int64 and np.array_equal(p, wperm), rev
    assert np.array_equal(rk.Array(xd), x, equal_nan=x.dtype.kind == "f")          # sort / sortperm leave x alone
    assert rk.sort_(xd) is xd
    assert np.array_equal(rk.Array(xd), orc.sort(x), equal_nan=x.dtype.kind == "f")


@pytest.mark.parametrize("dtype", TYPES)
@pytest.mark.parametrize("sz", [1, 2, 3, 4, 33, 333, 3333, 4096])
def test_reference_sizes_and_types(rk, orc, dtype, sz):
    _check(rk, orc, _rand(np.random.default_rng(sz), dtype, sz))


@pytest.mark.parametrize("dtype", TYPES)
@pytest.mark.parametrize("sz", [1, 2, 3, 4, 33, 333, 3333, 4096, 100_003])
def test_reference_lt_and_by(rk, orc, dtype, sz):
    """test/hip_rocarray/sorting.jl:20-26: `sort(xd; lt=!isless)`, `xd[sortperm(xd; lt=!isless)]`, `sort(xd; by=k -> 2k)`,
    `xd[sortperm(xd; by=k -> 2k)]` against the host's sorts (the reference compares values)."""
    x = _rand(np.random.default_rng(1000 + sz), dtype, sz)
    if np.dtype(dtype).kind == "i":
        x = (x // 4).astype(dtype)                              # 2k stays inside the type, as Julia's Int64 product does
    xd = rk.ROCArray(x)
    desc = np.sort(x)[::-1]
    assert np.array_equal(rk.Array(rk.sort(xd, lt=rk.not_isless)), desc)
    p = rk.Array(rk.sortperm(xd, lt=rk.not_isless))
    assert sorted(p.tolist()) == list(range(1, sz + 1)) and np.array_equal(x[p - 1], desc)
    by = lambda k: 2 * k                                        # noqa: E731
    asc = np.sort(x)
    assert np.array_equal(rk.Array(rk.sort(xd, by=by)), asc)
    p = rk.Array(rk.sortperm(xd, by=by))
    assert sorted(p.tolist()) == list(range(1, sz + 1)) and np.array_equal(x[p - 1], asc)
    assert np.array_equal(rk.Array(rk.sort(xd, by=lambda k: -k)), desc)       # a `by` that reverses
    assert np.array_equal(rk.Array(xd), x)
    y = rk.ROCArray(x)
    assert rk.sort_(y, by=by, rev=True) is y and np.array_equal(rk.Array(y), desc)
    with pytest.raises(NotImplementedError):
        rk.sort(xd, lt=lambda a, b: a < b)                      # any other comparator: the stock path


@pytest.mark.parametrize("dtype", TYPES)
@pytest.mark.parametrize("n", [4097, 65_537, 1_000_003])
def test_many_tiles(rk, orc, dtype, n):
    _check(rk, orc, _rand(np.random.default_rng(n), dtype, n))


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64])
def test_special_floats_and_stability(rk, orc, dtype):
    rng = np.random.default_rng(5)
    base = np.array([0.0, -0.0, np.nan, np.inf, -np.inf, 1.0, -1.0, 65504.0, -65504.0, 6e-8, -6e-8], dtype=dtype)
    x = rng.choice(base, 50_000)
    x[::7] = -x[::7]
    _check(rk, orc, x)


@pytest.mark.parametrize("dtype", [np.int16, np.int32, np.int64])
def test_small_range_integers_skip_passes(rk, orc, dtype):
    rng = np.random.default_rng(6)
    _check(rk, orc, rng.integers(-10, 11, 300_000).astype(dtype))                  # perf/array.jl:16 rand(-10:10, ...)
    _check(rk, orc, np.full(10_000, 7, dtype=dtype))                               # every pass skipped
    _check(rk, orc, (rng.integers(0, 2, 100_000) * 256).astype(dtype))             # only the second digit varies
    _check(rk, orc, np.arange(100_000, 0, -1).astype(dtype) if dtype != np.int16 else np.arange(30_000, 0, -1).astype(dtype))


def test_perf_suite_size_and_in_place_outputs(rk, orc):
    x = np.random.default_rng(7).random(512 * 1000).astype(np.float32)             # sort(gpu_vec), perf/array.jl:145
    _check(rk, orc, x)
    ix = rk.ROCArray(dims=(x.size,), dtype=np.int64)
    assert rk.sortperm_(ix, rk.ROCArray(x)) is ix
    assert np.array_equal(x[rk.Array(ix) - 1], np.sort(x))                         # y == xd[sortperm(xd)], sorting.jl:14


def test_full_size_sort(rk, orc):
    x = np.random.default_rng(8).standard_normal(1 << 24).astype(np.float32)
    got = rk.Array(rk.sort(rk.ROCArray(x)))
    assert np.array_equal(got, np.sort(x))
    k = np.random.default_rng(9).integers(-2**62, 2**62, 1 << 22, dtype=np.int64)
    p = rk.Array(rk.sortperm(rk.ROCArray(k), rev=True))
    assert np.array_equal(p, orc.sortperm(k, True))


# More than 256 tiles of 4096 keys: the sort counts the digits of every tile before each pass (no look-back).
LARGE = 1024 * 4096 + 4096 * 3 + 37


@pytest.mark.parametrize("dtype", TYPES)
def test_large_sorts_all_types(rk, orc, dtype):
    _check(rk, orc, _rand(np.random.default_rng(11), dtype, LARGE))


@pytest.mark.parametrize("dtype", [np.int16, np.int32, np.int64])
def test_large_small_range_integers(rk, orc, dtype):
    rng = np.random.default_rng(12)
    _check(rk, orc, rng.integers(-10, 11, LARGE).astype(dtype))                    # one pass: the range fits a digit
    _check(rk, orc, rng.integers(-300, 70_000 if dtype != np.int16 else 3_000, LARGE).astype(dtype))
    _check(rk, orc, np.full(LARGE, -5, dtype=dtype))                               # every pass skipped
    _check(rk, orc, (rng.integers(0, 2, LARGE) * 256).astype(dtype))               # low digit constant, not skipped


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_large_special_floats(rk, orc, dtype):
    rng = np.random.default_rng(13)
    base = np.array([0.0, -0.0, np.nan, np.inf, -np.inf, 1.0, -1.0, 65504.0, -65504.0, 6e-8, -6e-8], dtype=dtype)
    x = rng.choice(base, LARGE)
    x[::7] = -x[::7]
    _check(rk, orc, x)
    _check(rk, orc, (1.0 + rng.random(LARGE)).astype(dtype))                       # one binade: exponent digits constant


def test_large_unaligned_view(rk, orc):
    x = _rand(np.random.default_rng(14), np.float32, LARGE + 10)
    d = rk.ROCArray(x)
    v = d.view_range(4, LARGE + 6)                                                 # starts 12 bytes into the buffer
    assert np.array_equal(rk.Array(rk.sort(v)), orc.sort(x[3:LARGE + 6]))
    assert np.array_equal(rk.Array(rk.sortperm(v, rev=True)), orc.sortperm(x[3:LARGE + 6], True))
    rk.sort_(v)
    got = rk.Array(d)
    assert np.array_equal(got[3:LARGE + 6], orc.sort(x[3:LARGE + 6]))
    assert np.array_equal(got[:3], x[:3]) and np.array_equal(got[LARGE + 6:], x[LARGE + 6:])


@pytest.mark.parametrize("dtype", [np.int16, np.float32, np.float64])
def test_unaligned_views(rk, orc, dtype):
    # keys that start 1 .. 9 elements into a buffer: the vector body of the whole-array reads starts later
    x = _rand(np.random.default_rng(10), dtype, 70_010)
    d = rk.ROCArray(x)
    for first in (2, 3, 4, 6, 10):
        v = d.view_range(first, 70_005)
        want = orc.sort(x[first - 1:70_005])
        assert np.array_equal(rk.Array(rk.sort(v)), want)
        assert np.array_equal(rk.Array(rk.sortperm(v)), orc.sortperm(x[first - 1:70_005]))
    v = d.view_range(3, 70_001)
    rk.sort_(v, rev=True)
    got = rk.Array(d)
    assert np.array_equal(got[2:70_001], orc.sort(x[2:70_001], rev=True))
    assert np.array_equal(got[:2], x[:2]) and np.array_equal(got[70_001:], x[70_001:])      # neighbours untouched


def test_unsupported_forms(rk):
    xd = rk.ROCArray(np.arange(10, dtype=np.float32))
    with pytest.raises(rk.UnsupportedError):
        rk.sort(xd, lt=lambda a, b: a > b)
    with pytest.raises(rk.UnsupportedError):
        rk.sortperm(xd, by=lambda k: k if k > 0 else -k)        # control flow on the value: not traceable
    with pytest.raises(rk.UnsupportedError):
        rk.sort(rk.ROCArray(np.zeros((3, 4), dtype=np.float32)))
    with pytest.raises(rk.UnsupportedError):
        rk.sort(rk.ROCArray(np.zeros(5, dtype=np.uint8)))
    assert len(rk.sort(rk.ROCArray(np.zeros(0, dtype=np.float32)))) == 0


@pytest.mark.parametrize("dtype,utype", [(np.float32, np.uint32), (np.float64, np.uint64), (np.float16, np.uint16)])
@pytest.mark.parametrize("rev", [False, True])
def test_sort_keeps_nan_bit_patterns(rk, dtype, utype, rev):
    # sort!: the result is a permutation of the input bit for bit -- negative NaNs and payloads survive -- with the
    # non-NaN part in isless order and every NaN after it (before it with rev); sortperm: NaNs are equal keys, index order
    rng = np.random.default_rng(99)
    n = 300_000
    h = rng.standard_normal(n).astype(dtype)
    u = h.view(utype)
    nan_bits = {np.float32: [0xffc00001, 0x7fc12345, 0x7f800001, 0xff800001, 0x7fffffff, 0x7fc00000],
                np.float64: [0xfff8000000000001, 0x7ff8000000abcdef, 0x7ff0000000000001, 0xfff0000000000001, 0x7fffffffffffffff, 0x7ff8000000000000],
                np.float16: [0xfe01, 0x7e55, 0x7c01, 0xfc01, 0x7fff, 0x7e00]}[dtype]
    pos = rng.choice(n, 600, replace=False)
    for k, p_ in enumerate(pos):
        u[p_] = nan_bits[k % len(nan_bits)]
    h[rng.choice(n, 50)] = np.inf
    h[rng.choice(n, 50)] = -np.inf
    h[rng.choice(n, 50)] = -0.0
    d = rk.ROCArray(h.copy())
    rk.sort_(d, rev=rev)
    got = rk.Array(d)
    assert np.array_equal(np.sort(got.view(utype)), np.sort(h.view(utype)))            # a permutation of the bits
    nn = int(np.isnan(h).sum())
    body = got[nn:] if rev else got[:n - nn]
    tail = got[:nn] if rev else got[n - nn:]
    assert np.isnan(tail).all() and not np.isnan(body).any()
    want = np.sort(h[~np.isnan(h)])
    want = want[::-1] if rev else want
    assert np.array_equal(body, want) and np.array_equal(np.signbit(body), np.signbit(want))
    perm = rk.Array(rk.sortperm(rk.ROCArray(h), rev=rev)) - 1
    nan_part = perm[:nn] if rev else perm[n - nn:]
    assert np.array_equal(nan_part, np.flatnonzero(np.isnan(h)))                          # stable among the NaNs
    assert np.array_equal(np.sort(perm), np.arange(n))
