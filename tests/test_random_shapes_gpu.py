"""Differential test over seeded random shapes, dims, element types and operators: every family of the library against
the oracle on cases nobody chose by hand (the launch geometry of each kernel depends on the collapsed shape, so odd
extents and dims combinations reach paths that the fixed cases may miss).

Each case is printed (and flushed) before it runs, so that a failure names it.  Float32 sums rtol 1e-5 against the
Float64 host result (scans 1e-4, plus an absolute term for cancellation); integers, indices and moves bit-exact."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

EXTENTS = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 255, 256, 257, 513, 1000, 1024, 4097, 10_000]
DTYPES = [np.float32, np.float64, np.int32, np.int64]
MAX_ELEMS = 1 << 20
SEED = int(os.environ.get("RK_TEST_SEED", "0"))          # another value draws another set of cases


def _shape(rng):
    nd = int(rng.integers(1, 5))
    while True:
        shape = tuple(int(rng.choice(EXTENTS)) for _ in range(nd))
        if np.prod(shape, dtype=np.int64) <= MAX_ELEMS:
            return shape


def _dims(rng, nd):
    k = int(rng.integers(0, 4))
    if k == 0:
        return None
    pick = sorted(set(int(d) for d in rng.integers(1, nd + 1, size=k)))
    return pick[0] if len(pick) == 1 and rng.random() < 0.5 else tuple(pick)


def _data(rng, shape, dtype, small=False):
    if np.dtype(dtype).kind == "f":
        return rng.standard_normal(shape).astype(dtype)
    lim = 3 if small else 1000
    return rng.integers(-lim, lim + 1, shape).astype(dtype)


def _say(*what):
    print("CASE", *what, flush=True)
    sys.stdout.flush()


def _axes(dims, nd):
    if dims is None:
        return tuple(range(nd))
    return tuple(d - 1 for d in ((dims,) if isinstance(dims, int) else dims))


def test_random_reductions(rk, orc):
    rng = np.random.default_rng(1001 + SEED)
    for case in range(300):
        shape = _shape(rng)
        dtype = DTYPES[int(rng.integers(len(DTYPES)))]
        dims = _dims(rng, len(shape))
        op = ["add_sum", "add", "max", "min"][int(rng.integers(4))]
        f = ["identity", "abs2", "abs"][int(rng.integers(3))]
        _say("reduce", case, shape, np.dtype(dtype).name, dims, f, op)
        x = _data(rng, shape, dtype)
        got = rk.mapreduce(f, op, rk.ROCArray(x), dims=dims)
        want = orc.mapreduce(f, op, x, dims=dims)
        got = np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape)
        assert got.dtype == orc.reduce_eltype(op, dtype)          # the oracle itself accumulates floats in Float64
        if got.dtype.kind == "f" and op in ("add_sum", "add"):
            mag = float(np.max(orc.mapreduce("abs" if f != "abs2" else "abs2", op, x, dims=dims)))
            np.testing.assert_allclose(got, want, rtol=1e-5, atol=(1e-6 if dtype == np.float32 else 1e-12) * mag)
        elif got.dtype.kind == "f" and f == "abs2":
            np.testing.assert_allclose(got, want, rtol=1e-6)        # x * x rounds once in Float32, max / min pick exactly
        else:
            assert np.array_equal(got, want.astype(got.dtype))


NARROW = [np.int8, np.int16, np.uint16]


def test_random_narrow_integers(rk, orc):
    """Int8 / Int16 / UInt16: sums and products in the 64-bit type Base.add_sum / mul_prod widen them to, + / max / min
    in their own type (wrapping), findmax / findmin, all bit-exact."""
    rng = np.random.default_rng(1011 + SEED)
    for case in range(240):
        shape = _shape(rng)
        dtype = NARROW[int(rng.integers(len(NARROW)))]
        dims = _dims(rng, len(shape))
        op = ["add_sum", "add", "max", "min", "mul_prod"][int(rng.integers(5))]
        f = ["identity", "abs2", "abs"][int(rng.integers(3))]
        _say("narrow reduce", case, shape, np.dtype(dtype).name, dims, f, op)
        info = np.iinfo(dtype)
        if op == "mul_prod":
            x = rng.integers(max(info.min, -2), 3, shape).astype(dtype)
        else:
            x = rng.integers(info.min, info.max + 1, shape).astype(dtype)
        got = rk.mapreduce(f, op, rk.ROCArray(x), dims=dims)
        want = orc.mapreduce(f, op, x, dims=dims)
        got = np.asarray(got if dims is None else rk.Array(got)).reshape(want.shape)
        assert got.dtype == orc.reduce_eltype(op, dtype)
        assert np.array_equal(got, want.astype(got.dtype))
        if case % 3 == 0:
            y = rng.integers(max(info.min, -3), 4, shape).astype(dtype)          # few distinct values: the first-index rule decides
            dy = rk.ROCArray(y)
            for gpu, cpu in ((rk.findmax, orc.findmax), (rk.findmin, orc.findmin)):
                gv, gi = gpu(dy, dims=dims)
                ov, oi = cpu(y, dims=dims)
                if dims is None:
                    assert gv == ov and gi == oi
                else:
                    assert rk.Array(gv).dtype == y.dtype and np.array_equal(rk.Array(gv), ov)
                    assert np.array_equal(np.moveaxis(rk.Array(gi), 0, -1), oi)


def test_random_findminmax(rk, orc):
    rng = np.random.default_rng(1002 + SEED)
    for case in range(150):
        shape = _shape(rng)
        dtype = DTYPES[int(rng.integers(len(DTYPES)))]
        dims = _dims(rng, len(shape))
        _say("findminmax", case, shape, np.dtype(dtype).name, dims)
        x = _data(rng, shape, dtype, small=True)                  # few distinct values: the first-index rule decides
        dx = rk.ROCArray(x)
        for gpu, cpu in ((rk.findmax, orc.findmax), (rk.findmin, orc.findmin)):
            gv, gi = gpu(dx, dims=dims)
            ov, oi = cpu(x, dims=dims)
            if dims is None:
                assert gv == ov and gi == oi
            else:
                assert np.array_equal(rk.Array(gv), ov)
                assert np.array_equal(np.moveaxis(rk.Array(gi), 0, -1), oi)


def test_random_scans(rk, orc):
    rng = np.random.default_rng(1003 + SEED)
    for case in range(300):
        shape = _shape(rng)
        dtype = DTYPES[int(rng.integers(len(DTYPES)))]
        dim = int(rng.integers(1, len(shape) + 2))                # one past ndims: a copy with init folded in
        op = ["add", "add", "max", "min"][int(rng.integers(4))]
        inclusive = bool(rng.random() < 0.7)
        init = int(rng.integers(-5, 6)) if (not inclusive or rng.random() < 0.5) else None
        _say("scan", case, shape, np.dtype(dtype).name, dim, op, inclusive, init)
        x = _data(rng, shape, dtype)
        got = rk.Array(rk.accumulate(op, rk.ROCArray(x), dims=dim, init=init, inclusive=inclusive))
        want = orc.accumulate(op, x, dims=dim, init=init, inclusive=inclusive)
        # (the oracle scans floats in Float64; integer element types must agree exactly)
        assert got.dtype == (dtype if np.dtype(dtype).kind == "f" else want.dtype) and got.shape == want.shape
        if want.dtype.kind == "f" and op == "add":
            n = shape[dim - 1] if dim <= len(shape) else 1
            scale = float(np.abs(x).max()) * np.sqrt(n) + abs(init or 0)
            np.testing.assert_allclose(got, want, rtol=1e-4 if dtype == np.float32 else 1e-12,
                                       atol=(2e-6 if dtype == np.float32 else 1e-13) * scale * np.sqrt(n))
        else:
            assert np.array_equal(got, want.astype(got.dtype))


def test_random_narrow_scans(rk, orc):
    """Int8 / UInt8 / Int16 / UInt16 / Float16 scans over random shapes, dims, operators, init and inclusive: native in
    rk_accumulate (scanned in 32 bits, stored narrow).  Integers wrap in their own type and must agree bit for bit."""
    rng = np.random.default_rng(1007 + SEED)
    for case in range(200):
        shape = _shape(rng)
        dtype = [np.int8, np.uint8, np.int16, np.uint16, np.float16][int(rng.integers(5))]
        dt = np.dtype(dtype)
        dim = int(rng.integers(1, len(shape) + 2))
        op = ["add", "add", "max", "min", "mul"][int(rng.integers(5))]
        inclusive = bool(rng.random() < 0.7)
        init = int(rng.integers(0, 6)) if (not inclusive or rng.random() < 0.5) else None
        if op == "mul" and init is None and not inclusive:
            init = 1
        _say("narrow scan", case, shape, dt.name, dim, op, inclusive, init)
        if dt.kind == "f":
            x = (rng.random(shape) * 0.01).astype(dt) if op != "mul" else (1 + rng.random(shape) * 1e-3).astype(dt)
        else:
            info = np.iinfo(dt)
            x = rng.integers(info.min, info.max + 1, shape).astype(dt)
        got = rk.Array(rk.accumulate(op, rk.ROCArray(x), dims=dim, init=None if init is None else dt.type(init), inclusive=inclusive))
        want = orc.accumulate(op, x, dims=dim, init=None if init is None else dt.type(init), inclusive=inclusive)
        assert got.dtype == dt and got.shape == want.shape
        if dt.kind == "f":
            n = shape[dim - 1] if dim <= len(shape) else 1
            np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=4e-3, atol=1e-3 * (1 + abs(init or 0)) if op != "mul" else 4e-3 * n)
        else:
            assert np.array_equal(got, want.astype(dt))


def test_random_moves(rk, orc):
    rng = np.random.default_rng(1004 + SEED)
    for case in range(200):
        shape = _shape(rng)
        dtype = [np.float32, np.float64, np.int32, np.int64, np.uint8, np.int16][int(rng.integers(6))]
        nd = len(shape)
        x = rng.integers(0, 200, shape).astype(dtype)
        dx = rk.ROCArray(x)
        rdims = _dims(rng, nd)
        perm = tuple(int(p) + 1 for p in rng.permutation(nd))
        _say("move", case, shape, np.dtype(dtype).name, "reverse dims", rdims, "perm", perm)
        if rdims is None and nd > 1:
            rdims = tuple(range(1, nd + 1))                         # reverse(A; dims=:)
        got = rk.Array(rk.reverse(dx, dims=rdims)) if rdims is not None else rk.Array(rk.reverse(dx))
        assert np.array_equal(got, np.flip(x, axis=_axes(rdims, nd)))
        y = rk.ROCArray(x.copy())
        rk.reverse_(y, dims=rdims) if rdims is not None else rk.reverse_(y)
        assert np.array_equal(rk.Array(y), np.flip(x, axis=_axes(rdims, nd)))
        assert np.array_equal(rk.Array(rk.permutedims(dx, perm)), orc.permutedims(x, perm))


def test_random_broadcasts(rk):
    rng = np.random.default_rng(1005 + SEED)
    B = rk.broadcast
    lz = rk.lazy
    trees = [
        ("u + v * w", lambda u, v, w: u + v * w, lambda u, v, w: u + v * w),
        ("(u - v) / w", lambda u, v, w: (u - v) / w, lambda u, v, w: (u - v) / w),
        ("max(u, v) - min(v, w)", lambda u, v, w: B.max_(u, v) - B.min_(v, w), lambda u, v, w: np.maximum(u, v) - np.minimum(v, w)),
        ("u * u + v * v - w", lambda u, v, w: u * u + v * v - w, lambda u, v, w: u * u + v * v - w),
        ("ifelse(u > v, w, -w)", lambda u, v, w: B.ifelse(u > v, w, -w), lambda u, v, w: np.where(u > v, w, -w)),
        ("(u < v) & (v < w)", lambda u, v, w: (u < v) & (v < w), lambda u, v, w: (u < v) & (v < w)),
        ("abs(u - v) * 2 + w", lambda u, v, w: B.abs_(u - v) * np.float32(2) + w, lambda u, v, w: np.abs(u - v) * np.float32(2) + w),
    ]
    for case in range(250):
        shape = _shape(rng)
        nd = len(shape)
        name, gpu_f, cpu_f = trees[int(rng.integers(len(trees)))]
        hosts = []
        for _ in range(3):                                           # each operand: full, extruded in some dims, or a scalar
            kind = rng.random()
            if kind < 0.15:
                hosts.append(np.float32(rng.uniform(0.5, 1.5)))
            else:
                s = tuple(1 if (kind > 0.5 and rng.random() < 0.5) else n for n in shape)
                hosts.append((rng.random(s, dtype=np.float32) + np.float32(0.5)))
        if not any(isinstance(h, np.ndarray) and h.shape == shape for h in hosts):
            hosts[0] = rng.random(shape, dtype=np.float32) + np.float32(0.5)
        _say("broadcast", case, shape, name, [h.shape if isinstance(h, np.ndarray) else "scalar" for h in hosts])
        devs = [rk.ROCArray(h) if isinstance(h, np.ndarray) else h for h in hosts]
        got = rk.Array(rk.materialize(gpu_f(*(lz(d) for d in devs))))
        want = cpu_f(*hosts)
        assert got.shape == np.broadcast_shapes(*(h.shape if isinstance(h, np.ndarray) else () for h in hosts))
        if want.dtype == np.bool_:
            assert got.dtype == np.bool_ and np.array_equal(got, want)
        else:
            np.testing.assert_array_equal(got, want.astype(np.float32))      # un-fused Float32 arithmetic: bit for bit


def test_random_sorts_and_selections(rk, orc):
    rng = np.random.default_rng(1006 + SEED)
    sizes = EXTENTS + [65_536, 100_003, 300_000, (1 << 20) + 5]
    for case in range(80):
        n = int(rng.choice(sizes))
        dtype = [np.float32, np.float64, np.int32, np.int64, np.int16, np.float16][int(rng.integers(6))]
        rev = bool(rng.random() < 0.4)
        spread = [3, 1000, 2**15 - 1][int(rng.integers(3))]           # many ties / few ties
        _say("sort", case, n, np.dtype(dtype).name, "rev" if rev else "fwd", spread)
        if np.dtype(dtype).kind == "f":
            with np.errstate(over="ignore"):                          # Float16 overflows to +-Inf: fine, Inf sorts too
                x = (rng.standard_normal(n) * spread).astype(dtype)
            x[rng.random(n) < 0.01] = np.nan
            x[rng.random(n) < 0.01] = -0.0
            x[rng.random(n) < 0.01] = 0.0
        else:
            x = rng.integers(-spread, spread + 1, n).astype(dtype)
        dx = rk.ROCArray(x)
        got = rk.Array(rk.sort(dx, rev=rev))
        want = orc.sort(x, rev=rev)
        assert got.dtype == x.dtype and np.array_equal(got, want, equal_nan=True)
        if x.dtype.kind == "f":
            assert np.array_equal(np.signbit(got[~np.isnan(got)]), np.signbit(want[~np.isnan(want)]))
        assert np.array_equal(rk.Array(rk.sortperm(dx, rev=rev)), orc.sortperm(x, rev=rev))       # stable: one answer
    for case in range(80):
        shape = _shape(rng)
        density = [0.0, 0.001, 0.3, 0.9, 1.0][int(rng.integers(5))]
        _say("findall", case, shape, density)
        m = rng.random(shape) < density
        got = rk.Array(rk.findall(rk.ROCArray(m)))
        want = orc.findall(m)
        assert np.array_equal(got, want if len(shape) == 1 else want.T)
        assert rk.count(rk.ROCArray(m)) == int(m.sum())
