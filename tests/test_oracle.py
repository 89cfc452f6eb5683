"""Pins the CPU oracle (oracle/oracle.py and oracle/oracle_c.c) WITHOUT a GPU.

The reference tree holds no golden vectors for this path (its tests compare ROCArray against Array with
unseeded random inputs).  Each oracle function is therefore pinned by: the literal results the reference's
docs and tests do state, closed forms, brute-force sequential loops that restate Julia Base's definition
independently of the vectorised oracle, and invariants chosen so that a dropped term, a wrong sign, a
transposed operand or an off-by-one index fails.  The committed fixtures under tests/golden/ were written
by tests/golden/make_golden.py from the same oracle and guard against silent changes."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from oracle import oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


# ---- eltype rules ------------------------------------------------------------------------------------
def test_reduce_eltype_table():
    assert orc.reduce_eltype("add_sum", np.int32) == np.int64          # Base.add_sum widens
    assert orc.reduce_eltype("add_sum", np.int8) == np.int64
    assert orc.reduce_eltype("add_sum", np.uint32) == np.uint64
    assert orc.reduce_eltype("add_sum", np.bool_) == np.int64
    assert orc.reduce_eltype("add_sum", np.float32) == np.float32      # floats are never widened
    assert orc.reduce_eltype("add", np.int32) == np.int32              # plain + keeps the eltype
    assert orc.reduce_eltype("max", np.int32) == np.int32
    assert orc.accumulate_eltype("add", np.int32) == np.int32          # accumulate.jl:1-8: init = zero(eltype(A))
    assert orc.accumulate_eltype("add", np.bool_) == np.int64


# ---- literal results stated in the reference -------------------------------------------------------------
def test_reference_doctests():
    # docs/src/usage/arrays.md:85-96
    assert orc.sum_(np.arange(1, 101)) == 5050
    assert orc.mapreduce("abs2", "add", np.arange(1, 5)) == 30
    assert np.array_equal(orc.cumsum(np.array([1, 2, 3, 4])), [1, 3, 6, 10])
    # test/hip_rocarray/multi_gpu.jl:45,48
    assert orc.sum_(np.ones(16, dtype=np.int64)) == 16


# ---- reductions: closed forms and brute force --------------------------------------------------------------
def test_sum_closed_forms():
    n = 100_000
    assert orc.sum_(np.ones(n, dtype=np.float32)) == n
    assert orc.sum_(np.arange(1, n + 1, dtype=np.int32)) == n * (n + 1) // 2         # > 2^31: needs Int64
    assert orc.sum_(np.arange(1, n + 1, dtype=np.int32)).dtype == np.int64
    x = np.full(1 << 22, 1000, dtype=np.int32)
    assert orc.sum_(x) == (1 << 22) * 1000
    # plain + on Int32 wraps like Julia
    assert orc.mapreduce("identity", "add", np.full(3, 2**30, dtype=np.int32)) == np.int32(-(2**30))


def _brute_mapreduce(f, op, A, dims):
    """Sequential loops straight from the definition; `dims` 1-based tuple."""
    fmap = {"identity": lambda v: v, "abs2": lambda v: v * v, "abs": abs}[f]
    comb = {"add": lambda a, b: a + b, "mul": lambda a, b: a * b, "max": max, "min": min}[op]
    out_shape = tuple(1 if (d + 1) in dims else n for d, n in enumerate(A.shape))
    out = np.empty(out_shape, dtype=np.float64)
    seen = np.zeros(out_shape, dtype=bool)
    for idx in np.ndindex(*A.shape):
        o = tuple(0 if (d + 1) in dims else i for d, i in enumerate(idx))
        v = fmap(float(A[idx]))
        out[o] = comb(out[o], v) if seen[o] else v
        seen[o] = True
    return out


@pytest.mark.parametrize("shape,dims", [((5,), (1,)), ((4, 3), (1,)), ((4, 3), (2,)), ((3, 4, 5), (2,)), ((3, 4, 5), (1, 3)),
                                        ((2, 3, 4), (1, 2, 3)), ((4, 3), (3,))])
@pytest.mark.parametrize("f,op", [("identity", "add"), ("abs2", "add"), ("identity", "max"), ("abs", "min"), ("identity", "mul")])
def test_mapreduce_vs_brute_force(shape, dims, f, op):
    A = np.random.default_rng(1).integers(-5, 6, shape).astype(np.float64)
    got = orc.mapreduce(f, op, A, dims=dims)
    assert got.shape == tuple(1 if (d + 1) in dims else n for d, n in enumerate(A.shape))   # mapreduce.jl:95-107
    np.testing.assert_allclose(got, _brute_mapreduce(f, op, A, dims), rtol=1e-12)


def test_mapreduce_full_is_scalar_and_init_folds():
    A = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert orc.mapreduce("identity", "add", A).shape == ()
    assert orc.mapreduce("identity", "add", A, init=10) == 76
    assert orc.mapreduce("identity", "max", A, dims=1, init=100).tolist() == [[100.0] * 4]


def test_map_runs_in_the_element_type():
    """mapreduce(abs2, add_sum, x): abs2(x::Int16) is an Int16 and wraps, the widening happens in add_sum.  Worked by
    hand: abs2(Int16(300)) = 90000 - 65536 = 24464, abs2(Int16(-200)) = 40000 - 65536 = -25536, sum -1072 (Julia:
    sum(abs2, Int16[300, -200]) == -1072); abs(typemin(Int8)) == typemin(Int8); UInt16: 300^2 mod 2^16 = 24464."""
    r = orc.mapreduce("abs2", "add_sum", np.array([300, -200], dtype=np.int16))
    assert r.dtype == np.int64 and int(r) == -1072
    r = orc.mapreduce("abs", "max", np.array([-128, 5], dtype=np.int8))
    assert r.dtype == np.int8 and int(r) == 5                       # abs(-128) stays -128
    r = orc.mapreduce("abs2", "add_sum", np.array([300, 2], dtype=np.uint16))
    assert r.dtype == np.uint64 and int(r) == 24464 + 4
    r = orc.mapreduce("abs2", "add_sum", np.array([100000, 3], dtype=np.int32))
    assert r.dtype == np.int64 and int(r) == (100000 * 100000 - 2 * 2**32) + 9      # 10^10 wraps to 1410065408


def test_max_min_base_rules():
    assert np.isnan(orc.maximum(np.array([1.0, np.nan, 3.0])))               # NaN propagates (Base.max)
    assert np.isnan(orc.minimum(np.array([1.0, np.nan, 3.0])))
    m = orc.maximum(np.array([-0.0, 0.0]))
    assert m == 0 and not np.signbit(m)                                        # max(-0.0, 0.0) == 0.0
    assert np.signbit(orc.minimum(np.array([0.0, -0.0])))
    assert orc.julia_max(-0.0, 0.0) == 0 and not np.signbit(orc.julia_max(-0.0, 0.0))
    with pytest.raises(ValueError):
        orc.maximum(np.zeros(0))


# ---- findmax / findmin: sequential Base._rf_findmax loop ------------------------------------------------------
def _isless(a, b):
    an, bn = np.isnan(a), np.isnan(b)
    if an or bn:
        return (not an) and bn
    if a == b:
        return bool(np.signbit(a)) and not bool(np.signbit(b))
    return a < b


def _brute_findminmax(A, dims, want_max):
    """Base: findmax keeps (fm, im) unless isless(fm, fx); findmin unless isgreater(fm, fx), iterating in
    column-major order."""
    def isgreater(x, y):
        return _isless(x, y) if (np.isnan(x) or np.isnan(y)) else _isless(y, x)
    best = {}
    for lin in range(A.size):
        idx = np.unravel_index(lin, A.shape, order="F")
        o = tuple(0 if (d + 1) in dims else i for d, i in enumerate(idx))
        v = A[idx]
        if o not in best:
            best[o] = (v, idx)
        else:
            fm, im = best[o]
            take = _isless(fm, v) if want_max else isgreater(fm, v)
            if take:
                best[o] = (v, idx)
    return best


@pytest.mark.parametrize("want_max", [True, False])
@pytest.mark.parametrize("dims", [(1,), (2,), (1, 2), (3,)])
def test_findminmax_vs_sequential(want_max, dims):
    rng = np.random.default_rng(2)
    A = rng.integers(-2, 3, (5, 4, 3)).astype(np.float32)       # many ties
    A[1, 2, 0] = np.nan
    A[3, 2, 0] = np.nan
    A[0, 0, 1] = -0.0
    A[2, 0, 1] = 0.0
    vals, idx = orc.findminmax(A, want_max, dims=dims)
    for o, (v, ix) in _brute_findminmax(A, dims, want_max).items():
        got_v = vals[o]
        assert (np.isnan(got_v) and np.isnan(v)) or (got_v == v and np.signbit(got_v) == np.signbit(v))
        assert tuple(idx[o]) == tuple(i + 1 for i in ix)


def test_findmax_scalar_forms():
    v, i = orc.findmax(np.array([1.0, 7.0, 7.0, 3.0], dtype=np.float32))
    assert v == 7 and i == 2                                                     # first maximum, Int index for vectors
    v, i = orc.findmax(np.array([[1, 5], [7, 2]], dtype=np.int32))
    assert v == 7 and i == (2, 1)                                                # CartesianIndex(2, 1)
    v, i = orc.findmin(np.array([1.0, np.nan, 0.5]))
    assert np.isnan(v) and i == 2                                                # NaN wins in findmin too
    v, i = orc.findmax(np.array([-0.0, 0.0, -0.0]))
    assert i == 2 and not np.signbit(v)                                          # isless(-0.0, 0.0)


# ---- accumulate -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [0, 1, 2, 3, 10, 10_000, 16384, 16385])                 # test/core/rocarray_base.jl:195
def test_accumulate_sizes_vs_loop(n):
    x = np.random.default_rng(n).random(n)
    want = np.empty(n)
    acc = 0.0
    for i in range(n):
        acc = acc + x[i]
        want[i] = acc
    np.testing.assert_allclose(orc.accumulate("add", x), want, rtol=1e-13)
    init = 0.37
    np.testing.assert_allclose(orc.accumulate("add", x, init=init), want + init, rtol=1e-13)       # :198-200


@pytest.mark.parametrize("shape,dims", [((2,), 2), ((3, 4, 5), 2), ((1, 70, 50, 20), 3), ((3, 4, 5), 1), ((3, 4, 5), 3)])
def test_accumulate_dims_vs_loop(shape, dims):                                                      # :204-213
    x = np.random.default_rng(3).integers(-10**6, 10**6, shape, dtype=np.int64)
    want = x.copy()
    if dims <= x.ndim:
        for idx in np.ndindex(*shape):
            if idx[dims - 1] > 0:
                prev = list(idx)
                prev[dims - 1] -= 1
                want[idx] = want[tuple(prev)] + x[idx]
    assert np.array_equal(orc.accumulate("add", x, dims=dims), want)


def test_accumulate_int32_wraps_and_keeps_eltype():
    x = np.full(10, 2**30, dtype=np.int32)
    got = orc.cumsum(x)
    assert got.dtype == np.int32
    want = [((k + 1) * 2**30 + 2**31) % 2**32 - 2**31 for k in range(10)]                           # mod 2^32
    assert got.tolist() == want


def test_accumulate_exclusive_and_ops():
    x = np.array([3, 1, 4, 1, 5], dtype=np.int64)
    assert orc.accumulate("add", x, init=10, inclusive=False).tolist() == [10, 13, 14, 18, 19]
    assert orc.accumulate("mul", x).tolist() == [3, 3, 12, 12, 60]
    assert orc.accumulate("max", x).tolist() == [3, 3, 4, 4, 5]
    assert orc.accumulate("min", x, init=2).tolist() == [2, 1, 1, 1, 1]
    assert orc.cumprod(np.array([1.5, 2.0])).tolist() == [1.5, 3.0]                                  # :224
    # a dim beyond ndims: every element is a line of length one, out[i] = op(init, x[i]) for every operator
    assert orc.accumulate("min", x, dims=2, init=2).tolist() == [2, 1, 2, 1, 2]
    assert orc.accumulate("max", x, dims=2, init=2).tolist() == [3, 2, 4, 2, 5]
    assert orc.accumulate("mul", x, dims=3, init=2).tolist() == [6, 2, 8, 2, 10]
    assert orc.accumulate("add", x, dims=2, init=2, inclusive=False).tolist() == [2, 2, 2, 2, 2]


def test_findall_matches_definition():
    m = np.array([[True, False, True], [False, False, True]])
    assert orc.findall(m).tolist() == [[1, 1], [1, 3], [2, 3]]                # column-major order of CartesianIndices
    v = np.array([False, True, True, False, True])
    assert orc.findall(v).tolist() == [2, 3, 5]


# ---- broadcast ------------------------------------------------------------------------------------------------------
def test_broadcast_shape_rule_is_julias():
    assert orc.broadcast_shape((2, 3), (1, 3)) == (2, 3)                        # rocarray_broadcast.jl:19
    assert orc.broadcast_shape((2, 3), (2,)) == (2, 3)                          # :20 (vector extrudes along dim 2)
    assert orc.broadcast_shape((3,), (3, 4, 5)) == (3, 4, 5)
    with pytest.raises(ValueError):
        orc.broadcast_shape((2, 3), (3,))                                       # NumPy would accept this, Julia does not


def test_broadcast_elementwise_loops():
    rng = np.random.default_rng(4)
    a = 0.5
    x, y, w = (rng.standard_normal((3, 4, 2)) for _ in range(3))
    got = orc.broadcast_axpby_exp(a, x, y, w)
    for idx in np.ndindex(3, 4, 2):
        assert got[idx] == pytest.approx(a * x[idx] + y[idx] * np.exp(w[idx]), rel=1e-15)
    A, r, c = rng.random((4, 3)), rng.random((1, 3)), rng.random((4, 1))
    got = orc.broadcast_rowcol(A, r, c)
    for i in range(4):
        for j in range(3):
            assert got[i, j] == A[i, j] + r[0, j] * c[i, 0]
    # vector extruded along dim 2 (Julia) -- not what NumPy's trailing alignment would do
    z = orc.broadcast_eval([("arg", 0), ("arg", 1), "add"], [A, np.arange(4.0)])
    assert z[2, 1] == A[2, 1] + 2.0
    assert orc.broadcast_eval([("arg", 0), ("arg", 1), ("arg", 2), "fma"], [2.0, 3.0, 4.0]) == 10.0


# ---- volumerhs -----------------------------------------------------------------------------------------------------------
def _vr_inputs(ne, seed=4):
    c = orc.config_inputs("volumerhs", scale=ne / 4000)
    assert c["Q"].shape[4] == ne
    return c


def test_volumerhs_two_restatements_agree():
    c = _vr_inputs(3)
    c["rhs"] = np.random.default_rng(9).standard_normal(c["rhs"].shape)
    a = orc.volumerhs(c["rhs"], c["Q"], c["vgeo"], c["gravity"], c["D"])
    b = orc.volumerhs_loops(c["rhs"], c["Q"], c["vgeo"], c["gravity"], c["D"])
    np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-10)


def test_volumerhs_constant_state_invariant():
    """If the columns of D sum to zero and Q, metrics are constant inside an element, every derivative term
    vanishes and only -MJI*MJ*rho*g is left on the W equation (perf/volumerhs.jl:140)."""
    ne = 2
    Q = np.empty((5, 5, 5, 5, ne))
    for s, v in enumerate((1.2, 0.3, -0.2, 0.1, 25.0)):
        Q[:, :, :, s, :] = v
    vgeo = np.empty((5, 5, 5, 14, ne))
    for f in range(14):
        vgeo[:, :, :, f, :] = 0.9 + 0.01 * f
    D = np.random.default_rng(6).standard_normal((5, 5))
    D -= D.mean(axis=0, keepdims=True)
    out = orc.volumerhs(np.zeros_like(Q), Q, vgeo, 9.81, D)
    want = np.zeros_like(Q)
    want[:, :, :, 3, :] = -vgeo[0, 0, 0, 10, 0] * vgeo[0, 0, 0, 9, 0] * 1.2 * 9.81
    np.testing.assert_allclose(out, want, atol=1e-11)
    # transposing D breaks the invariant: the oracle distinguishes D[n, i] from D[i, n]
    assert np.abs(orc.volumerhs(np.zeros_like(Q), Q, vgeo, 9.81, D.T) - want).max() > 1e-3


def test_volumerhs_linear_in_D_and_additive_in_rhs():
    c = _vr_inputs(2)
    z = np.zeros_like(c["rhs"], dtype=np.float64)
    D1 = c["D"].astype(np.float64)
    D2 = np.random.default_rng(7).random((5, 5))
    f = lambda D: orc.volumerhs(z, c["Q"], c["vgeo"], c["gravity"], D)
    src = f(np.zeros((5, 5)))                                                # gravity source term only
    np.testing.assert_allclose(f(D1 + 2 * D2) - src, (f(D1) - src) + 2 * (f(D2) - src), rtol=1e-10, atol=1e-9)
    r0 = np.random.default_rng(8).standard_normal(z.shape)
    np.testing.assert_allclose(orc.volumerhs(r0, c["Q"], c["vgeo"], c["gravity"], D1), r0 + f(D1), rtol=1e-12)


def test_volumerhs_single_node_by_hand():
    """One node carries data; D = identity picks F, G, H at the node itself.  Worked by hand from
    perf/volumerhs.jl:92-128 with rho=2, U=V=W=1 -> 0, E=10, z=0, all metric derivatives 1, MJ=MJI=1."""
    Q = np.zeros((5, 5, 5, 5, 1))
    Q[..., 0, :] = 2.0       # rho everywhere (avoid 1/0), momentum zero
    Q[..., 4, :] = 10.0      # E
    vgeo = np.zeros((5, 5, 5, 14, 1))
    vgeo[..., 0:9, :] = 1.0
    vgeo[..., 9, :] = 1.0
    vgeo[..., 10, :] = 1.0
    out = orc.volumerhs(np.zeros_like(Q), Q, vgeo, 0.0, np.eye(5))
    # P = 0.4 * E = 4; fluxes: only the pressure terms survive: flux_U_x = flux_V_y = flux_W_z = P.
    # F_U = xi_x*P = 4, F_V = xi_y*P = 4, F_W = 4 (same for G and H); identity D sums F + G + H = 12.
    assert np.allclose(out[..., 0, 0], 0) and np.allclose(out[..., 4, 0], 0)
    for s in (1, 2, 3):
        assert np.allclose(out[..., s, 0], 12.0)


# ---- C restatement vs NumPy oracle ------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def corc():
    so = os.path.join(ROOT, "oracle", "liboracle_c.so")
    if not os.path.exists(so):
        import subprocess
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-s"], check=True)
    lib = C.CDLL(so)
    lib.orc_sum_f32.restype = C.c_double
    lib.orc_sum_i32.restype = C.c_int64
    lib.orc_maximum_f32.restype = C.c_float
    return lib


def _p(a):
    return C.c_void_p(a.ctypes.data)


@pytest.mark.parametrize("threads", [1, 4])
def test_c_oracle_matches_numpy_oracle(corc, threads):
    rng = np.random.default_rng(11)
    x = rng.random(300_001, dtype=np.float32)
    np.testing.assert_allclose(corc.orc_sum_f32(_p(x), C.c_int64(x.size), threads), orc.sum_(x), rtol=1e-5)
    xi = rng.integers(-1000, 1001, 300_001, dtype=np.int32)
    assert corc.orc_sum_i32(_p(xi), C.c_int64(xi.size), threads) == orc.sum_(xi)
    m, n = 301, 203
    A = np.asfortranarray(rng.standard_normal((m, n), dtype=np.float32))
    o1, o2 = np.empty(n, dtype=np.float32), np.empty(m, dtype=np.float32)
    corc.orc_abs2sum_dims1_f32(_p(A), C.c_int64(m), C.c_int64(n), _p(o1), threads)
    corc.orc_abs2sum_dims2_f32(_p(A), C.c_int64(m), C.c_int64(n), _p(o2), threads)
    np.testing.assert_allclose(o1, orc.mapreduce("abs2", "add", A, dims=1).ravel(), rtol=1e-5)
    np.testing.assert_allclose(o2, orc.mapreduce("abs2", "add", A, dims=2).ravel(), rtol=1e-5)
    A[5, 7] = np.nan
    A[9, 7] = np.nan
    A[3, 8] = A[1, 8] = A[:, 8].max() + 1
    vals, rows = np.empty(n, dtype=np.float32), np.empty(n, dtype=np.int64)
    corc.orc_findmax_dims1_f32(_p(A), C.c_int64(m), C.c_int64(n), _p(vals), _p(rows), threads)
    ov, oi = orc.findmax(A, dims=1)
    assert np.array_equal(vals, ov.ravel(), equal_nan=True) and np.array_equal(rows, oi[0, :, 0])
    out = np.empty_like(xi)
    corc.orc_cumsum_i32(_p(xi), C.c_int64(xi.size), _p(out))
    assert np.array_equal(out, orc.cumsum(xi))
    B = np.asfortranarray(rng.random((m, n), dtype=np.float32))
    Bo = np.empty_like(B)
    corc.orc_cumsum_dims1_f32(_p(B), C.c_int64(m), C.c_int64(n), _p(Bo), threads)
    np.testing.assert_allclose(Bo, orc.cumsum(B, dims=1), rtol=1e-4)
    Bo2 = np.empty_like(B)
    corc.orc_cumsum_dims2_f32(_p(B), C.c_int64(m), C.c_int64(n), _p(Bo2), threads)
    np.testing.assert_allclose(Bo2, np.cumsum(B.astype(np.float64), axis=1), rtol=1e-4)
    # maximum: Base.max rules -- plain values, a planted NaN, and +0.0 against -0.0
    assert corc.orc_maximum_f32(_p(x), C.c_int64(x.size), threads) == x.max()
    xn = x.copy()
    xn[123_456] = np.nan
    assert np.isnan(corc.orc_maximum_f32(_p(xn), C.c_int64(xn.size), threads))
    zs = np.array([-0.0, 0.0, -0.0], dtype=np.float32)
    assert not np.signbit(np.float32(corc.orc_maximum_f32(_p(zs), C.c_int64(3), 1)))
    y, w = rng.standard_normal(x.size, dtype=np.float32), rng.standard_normal(x.size, dtype=np.float32)
    z = np.empty_like(x)
    corc.orc_bcast_axpby_exp_f32(C.c_float(0.5), _p(x), _p(y), _p(w), _p(z), C.c_int64(x.size), threads)
    np.testing.assert_allclose(z, orc.broadcast_axpby_exp(0.5, x, y, w), rtol=1e-5, atol=1e-6)
    r, c = rng.random((1, n), dtype=np.float32), rng.random((m, 1), dtype=np.float32)
    Cm = np.empty_like(A)
    corc.orc_bcast_rowcol_f32(_p(B), _p(r), _p(c), _p(Cm), C.c_int64(m), C.c_int64(n), threads)
    assert np.array_equal(Cm, B + r * c)
    cfg = orc.config_inputs("volumerhs", scale=6 / 4000)
    Q, vg, D = (np.asfortranarray(cfg[k]) for k in ("Q", "vgeo", "D"))
    rhs = np.asfortranarray(rng.standard_normal(Q.shape).astype(np.float32))
    want = orc.volumerhs(rhs, Q, vg, cfg["gravity"], D)
    corc.orc_volumerhs_f32(_p(rhs), _p(Q), _p(vg), C.c_float(9.81), _p(D), C.c_int64(Q.shape[4]), threads)
    np.testing.assert_allclose(rhs, want, rtol=1e-4, atol=1e-4 * np.abs(want).max())


# ---- committed fixtures ---------------------------------------------------------------------------------------------------------
def test_golden_fixtures_unchanged():
    with open(os.path.join(HERE, "golden", "oracle_golden.json")) as fh:
        gold = json.load(fh)
    from tests.golden.make_golden import compute
    now = compute()
    assert set(now) == set(gold)
    for k in gold:
        np.testing.assert_allclose(np.array(now[k], dtype=np.float64), np.array(gold[k], dtype=np.float64), rtol=1e-12, err_msg=k)


def test_reverse_matches_definition(orc):
    # element-by-element definition of reverse.jl:73-80: y[ref - idx on flipped dims] = x[idx]
    rng = np.random.default_rng(7)
    x = rng.integers(-100, 100, (3, 4, 5)).astype(np.int16)
    for dims in (None, 1, 2, 3, (1, 3), (2, 3), (1, 2, 3)):
        flip = {1, 2, 3} if dims is None else ({dims} if isinstance(dims, int) else set(dims))
        want = np.empty_like(x)
        for i in range(3):
            for j in range(4):
                for k in range(5):
                    want[2 - i if 1 in flip else i, 3 - j if 2 in flip else j, 4 - k if 3 in flip else k] = x[i, j, k]
        assert np.array_equal(orc.reverse(x, dims=dims), want)
    v = np.arange(1, 11)
    assert orc.reverse(v).tolist() == list(range(10, 0, -1))
    assert orc.reverse(v, 3, 6).tolist() == [1, 2, 6, 5, 4, 3, 7, 8, 9, 10]          # Base: reverse(1:10 |> collect, 3, 6)
    assert orc.reverse(v, 4).tolist() == [1, 2, 3, 10, 9, 8, 7, 6, 5, 4]


def test_permutedims_matches_definition(orc):
    rng = np.random.default_rng(8)
    x = rng.integers(-100, 100, (2, 3, 4)).astype(np.int32)
    for perm in ((1, 2, 3), (2, 1, 3), (3, 1, 2), (3, 2, 1), (1, 3, 2), (2, 3, 1)):
        out = orc.permutedims(x, perm)
        assert out.shape == tuple(x.shape[p - 1] for p in perm)
        for i in range(2):
            for j in range(3):
                for k in range(4):
                    idx = (i, j, k)
                    assert out[tuple(idx[p - 1] for p in perm)] == x[i, j, k]
    m = np.array([[1, 2, 3], [4, 5, 6]])
    assert orc.permutedims(m, (2, 1)).tolist() == [[1, 4], [2, 5], [3, 6]]       # Base docs: permutedims of a matrix


def test_sort_matches_isless_insertion_sort(orc):
    # Base.isless restated as a comparison, then a textbook stable insertion sort: pins order of signed zeros,
    # NaNs, infinities and the stability of sortperm (also with rev=true)
    import math

    def isless(a, b):
        if isinstance(a, float) or isinstance(b, float):
            if math.isnan(a):
                return False
            if math.isnan(b):
                return True
            if a == b == 0.0:
                return math.copysign(1.0, a) < math.copysign(1.0, b)
        return a < b

    def insertion_perm(v, rev):
        lt = (lambda a, b: isless(b, a)) if rev else isless
        p = []
        for i, e in enumerate(v):
            k = len(p)
            while k > 0 and lt(e, v[p[k - 1]]):
                k -= 1
            p.insert(k, i)
        return [i + 1 for i in p]

    rng = np.random.default_rng(9)
    specials = [0.0, -0.0, np.nan, np.inf, -np.inf, 1.5, -1.5, 0.0, -0.0, np.nan, 1.5]
    for dtype in (np.float16, np.float32, np.float64):
        v = np.array(specials + list(rng.integers(-3, 4, 20).astype(float)), dtype=dtype)
        for rev in (False, True):
            assert orc.sortperm(v, rev).tolist() == insertion_perm([float(e) for e in v], rev)
            s = orc.sort(v, rev)
            assert np.array_equal(s.view(f"u{v.itemsize}"), v[np.array(insertion_perm([float(e) for e in v], rev)) - 1].view(f"u{v.itemsize}"))
    for dtype in (np.int16, np.int32, np.int64):
        info = np.iinfo(dtype)
        v = np.array([0, -1, info.min, info.max, 5, 5, -1, info.min] + list(rng.integers(-5, 6, 20)), dtype=dtype)
        for rev in (False, True):
            assert orc.sortperm(v, rev).tolist() == insertion_perm([int(e) for e in v], rev)
    x = rng.standard_normal(1000).astype(np.float32)
    assert np.array_equal(orc.sort(x), np.sort(x)) and np.array_equal(orc.sort(x, rev=True), np.sort(x)[::-1])
    assert orc.sort(np.array([3, 1, 2])).tolist() == [1, 2, 3]
    assert orc.sortperm(np.array([3, 1, 2])).tolist() == [2, 3, 1]                 # Base docs: sortperm([3, 1, 2])


def test_bitwise_scans_against_a_sequential_loop():
    """accumulate(&, A), accumulate(|, A), accumulate(xor, A): pinned by the definition itself, a sequential loop over
    every line, for signed, unsigned and Bool element types, with and without init, inclusive and exclusive, and
    along a dim beyond ndims (a copy with init folded in)."""
    rng = np.random.default_rng(77)
    py = {"and": lambda a, b: a & b, "or": lambda a, b: a | b, "xor": lambda a, b: a ^ b}
    for dtype in (np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64, np.bool_):
        dt = np.dtype(dtype)
        shape = (5, 7, 3)
        x = (rng.random(shape) < 0.6) if dt == np.bool_ else rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, shape, dtype=dt, endpoint=True)
        for op in ("and", "or", "xor"):
            assert orc.accumulate_eltype(op, dt) == dt                       # Bool stays Bool under these
            for dims in (1, 2, 3, 4):
                for init, inclusive in ((None, True), (x.reshape(-1)[3], True), (x.reshape(-1)[5], False), (None, False)):
                    got = orc.accumulate(op, x, dims=dims, init=init, inclusive=inclusive)
                    assert got.dtype == dt and got.shape == shape
                    neutral = (True if dt == np.bool_ else dt.type(-1 if dt.kind == "i" else np.iinfo(dt).max)) if op == "and" else dt.type(0)
                    seed = neutral if init is None else init
                    want = np.empty_like(x)
                    moved = np.moveaxis(x, dims - 1, 0) if dims <= 3 else x[None]
                    wmoved = np.moveaxis(want, dims - 1, 0) if dims <= 3 else want[None]
                    for idx in np.ndindex(moved.shape[1:]):
                        run = seed
                        for k in range(moved.shape[0]):
                            v = moved[(k,) + idx]
                            if inclusive:
                                run = py[op](run, v)
                                wmoved[(k,) + idx] = run
                            else:
                                wmoved[(k,) + idx] = run
                                run = py[op](run, v)
                    assert np.array_equal(got, want), (dt, op, dims, init, inclusive)
