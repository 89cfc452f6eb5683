"""GPU parity of fused broadcast against the oracle, through the C ABI.

Float32 arithmetic is not contracted, so +,-,*,/ match a Float32 host evaluation bit for bit; results
that involve exp/log/sin/... are compared with the mixed tolerance
|got - ref| <= 1e-6 * (|a x| + |y e^w|) + 1e-5 * |ref| against Float64."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _rng(seed):
    return np.random.default_rng(seed)


def _axpby_check(rk, orc, a, x, y, w):
    z = rk.ROCArray(dims=x.shape, dtype=np.float32)
    L = rk.lazy
    out = rk.materialize_(z, a * L(rk.ROCArray(x)) + L(rk.ROCArray(y)) * rk.broadcast.exp(L(rk.ROCArray(w))))
    assert out is z
    got = rk.Array(z).astype(np.float64)
    ref = orc.broadcast_axpby_exp(a, x, y, w)
    x64, y64, w64 = (v.astype(np.float64) for v in (x, y, w))
    bound = 1e-6 * (np.abs(float(a) * x64) + np.abs(y64 * np.exp(w64))) + 1e-5 * np.abs(ref)
    assert np.all(np.abs(got - ref) <= bound)


@pytest.mark.parametrize("shape", [(1,), (5,), (64,), (1000,), (4096,), (33, 7), (32, 16, 8), (100, 100, 10), (3, 5, 7, 2)])
def test_axpby_exp_shapes(rk, orc, shape):
    rng = _rng(40)
    x, y, w = (rng.standard_normal(shape, dtype=np.float32) for _ in range(3))
    _axpby_check(rk, orc, np.float32(0.5), x, y, w)


def test_config4a_full_size(rk, orc):
    c = orc.config_inputs("bcast_axpby_exp")
    _axpby_check(rk, orc, c["a"], c["x"], c["y"], c["w"])


@pytest.mark.parametrize("m,n", [(4, 4), (5, 3), (64, 64), (100, 1000), (1000, 100), (1024, 37), (3, 100_000)])
def test_rowcol(rk, orc, m, n):
    rng = _rng(41)
    u = lambda *s: (rng.random(s, dtype=np.float32) * 2 - 1).astype(np.float32)
    A, r, c = u(m, n), u(1, n), u(m, 1)
    C = rk.ROCArray(dims=(m, n), dtype=np.float32)
    L = rk.lazy
    rk.materialize_(C, L(rk.ROCArray(A)) + L(rk.ROCArray(r)) * L(rk.ROCArray(c)))
    got = rk.Array(C)
    assert np.array_equal(got, A + r * c)            # un-contracted Float32: bit-exact with a Float32 host evaluation
    np.testing.assert_allclose(got, orc.broadcast_rowcol(A, r, c), rtol=1e-6, atol=1e-7)


def test_config4b_full_size(rk, orc):
    c = orc.config_inputs("bcast_rowcol")
    L = rk.lazy
    C = rk.materialize(L(rk.ROCArray(c["A"])) + L(rk.ROCArray(c["r"])) * L(rk.ROCArray(c["c"])))
    assert np.array_equal(rk.Array(C), c["A"] + c["r"] * c["c"])


def test_reference_broadcast_cases(rk, orc):
    """test/core/rocarray_broadcast.jl:5-28, the cases inside the enumerated op set."""
    L, B = rk.lazy, rk.broadcast
    rng = _rng(42)
    x = rng.random((3, 3))
    d = rk.ROCArray(x.copy())
    assert np.array_equal(rk.Array(rk.fill_(d, 1)), np.ones((3, 3)))                      # fill!(x, 1)
    a, b = rng.random((2, 3)), rng.random((2, 3))
    assert np.array_equal(rk.Array(rk.materialize(L(rk.ROCArray(a)) + L(rk.ROCArray(b)))), a + b)   # map(+, x, y)
    np.testing.assert_allclose(rk.Array(rk.materialize(B.sin(L(rk.ROCArray(a))))), np.sin(a), rtol=1e-13)
    np.testing.assert_allclose(rk.Array(rk.materialize(B.log(L(rk.ROCArray(a))) + 1)), np.log(a) + 1, rtol=1e-13)
    assert np.array_equal(rk.Array(rk.materialize(2 * L(rk.ROCArray(a)))), 2 * a)          # 2x
    np.testing.assert_allclose(rk.Array(rk.materialize(L(rk.ROCArray(a)) ** 3)), a ** 3, rtol=1e-13)
    np.testing.assert_allclose(rk.Array(rk.materialize(L(rk.ROCArray(a)) ** np.pi)), a ** np.pi, rtol=1e-13)
    # (2,3) .+ (1,3): row extrusion                                                         :19
    r = rng.random((1, 3))
    assert np.array_equal(rk.Array(rk.materialize(L(rk.ROCArray(a)) + L(rk.ROCArray(r)))), a + r)
    # z .= x .+ y with y a vector extruded along dim 2                                      :20
    y = rng.random(2)
    z = rk.ROCArray(rng.random((2, 3)))
    rk.materialize_(z, L(rk.ROCArray(a)) + L(rk.ROCArray(y)))
    assert np.array_equal(rk.Array(z), a + y[:, None])
    # Int + Float64 promotes to Float64                                                     :22
    got = rk.materialize(L(rk.ROCArray(np.array([1, 2, 3]))) + L(rk.ROCArray(np.array([1.0, 2.0, 3.0]))))
    assert got.dtype == np.float64 and np.array_equal(rk.Array(got), [2, 4, 6])
    # Ref(1) scalar operand: log.(x .+ xs)                                                  :38
    np.testing.assert_allclose(rk.Array(rk.materialize(B.log(1 + L(rk.ROCArray(x))))), np.log(1 + x), rtol=1e-13)
    # benchmark broadcast: gpu_mat .= 0f0 (perf/array.jl:67)
    g = rk.ROCArray(rng.random((512, 1000), dtype=np.float32))
    rk.fill_(g, np.float32(0))
    assert not rk.Array(g).any()


def test_interpreter_general_expression(rk, orc):
    L, B = rk.lazy, rk.broadcast
    rng = _rng(43)
    a, b, c = (rng.random((37, 11), dtype=np.float32) + np.float32(0.5) for _ in range(3))
    col = rng.random((37, 1), dtype=np.float32)
    da, db, dc, dcol = (rk.ROCArray(v) for v in (a, b, c, col))
    expr = B.sqrt(L(da) * L(db) + L(dc)) / (L(dcol) + np.float32(2)) - B.max_(L(da), L(db)) * B.abs2(L(dc))
    got = rk.Array(rk.materialize(expr))
    post = [("arg", 0), ("arg", 1), "mul", ("arg", 2), "add", "sqrt", ("arg", 3), ("arg", 4), "add", "div",
            ("arg", 0), ("arg", 1), "max", ("arg", 2), "abs2", "mul", "sub"]
    ref = orc.broadcast_eval(post, [a, b, c, col, np.float32(2)])
    assert got.dtype == np.float32
    np.testing.assert_allclose(got, ref, rtol=2e-6, atol=1e-6)
    # muladd and deep nesting on vector-aligned shapes
    x = rng.random((64, 32), dtype=np.float32)
    dx = rk.ROCArray(x)
    e2 = B.muladd(L(dx), L(dx), B.exp(-(L(dx)))) + B.tanh(L(dx)) * B.cos(L(dx)) - B.inv(L(dx) + np.float32(1))
    ref2 = x.astype(np.float64) ** 2 + np.exp(-x.astype(np.float64)) + np.tanh(x) * np.cos(x) - 1 / (x.astype(np.float64) + 1)
    np.testing.assert_allclose(rk.Array(rk.materialize(e2)), ref2, rtol=1e-5, atol=1e-6)


def test_dimension_mismatch(rk):
    L = rk.lazy
    a = rk.ROCArray(np.zeros((2, 3), dtype=np.float32))
    b = rk.ROCArray(np.zeros((3, 3), dtype=np.float32))
    with pytest.raises(rk.DimensionMismatch):
        rk.materialize(L(a) + L(b))
    with pytest.raises(rk.DimensionMismatch):
        rk.materialize_(rk.ROCArray(np.zeros((2,), dtype=np.float32)), L(a) + 1.0)


def test_unaligned_and_f64(rk, orc):
    L = rk.lazy
    x = _rng(44).random(10_001)
    d = rk.ROCArray(x)
    v = d.view_range(2, 10_001)
    got = rk.materialize(L(v) * 3.0 + 1.0)
    assert got.dtype == np.float64
    assert np.array_equal(rk.Array(got), x[1:] * 3.0 + 1.0)


def test_integer_programs_are_exact_and_wrap(rk):
    # all-integer + - * max min abs compute in Int64 and keep Julia's result eltype; Int32 results wrap
    rng = np.random.default_rng(50)
    L = rk.lazy
    a32 = rng.integers(-2**31, 2**31 - 1, (300, 70), dtype=np.int32)
    b32 = rng.integers(-2**31, 2**31 - 1, (300, 70), dtype=np.int32)
    got = rk.materialize(L(rk.ROCArray(a32)) + L(rk.ROCArray(b32)) * L(rk.ROCArray(a32)))
    assert got.dtype == np.int32
    with np.errstate(over="ignore"):
        assert np.array_equal(rk.Array(got), a32 + b32 * a32)                   # NumPy wraps Int32 like Julia
    a64 = rng.integers(-2**62, 2**62, 100_003, dtype=np.int64)
    b64 = rng.integers(-2**62, 2**62, 100_003, dtype=np.int64)
    got = rk.materialize(L(rk.ROCArray(a64)) * 3 - L(rk.ROCArray(b64)))         # beyond 2^53: a Float64 detour would lose bits
    assert got.dtype == np.int64
    with np.errstate(over="ignore"):
        assert np.array_equal(rk.Array(got), a64 * 3 - b64)
    got = rk.materialize(rk.broadcast.max_(L(rk.ROCArray(a64)), L(rk.ROCArray(b64))) + rk.broadcast.abs_(L(rk.ROCArray(a32[:, 0].astype(np.int64)[:1]))))
    assert np.array_equal(rk.Array(got), np.maximum(a64, b64) + abs(np.int64(a32[0, 0])))
    # Int32 matrix .+ Int64 column: promotes to Int64; row/column extrusion
    col = rng.integers(-1000, 1000, (300, 1), dtype=np.int64)
    got = rk.materialize(L(rk.ROCArray(a32)) + L(rk.ROCArray(col)))
    assert got.dtype == np.int64 and np.array_equal(rk.Array(got), a32.astype(np.int64) + col)
    # gpu_mat_ints .+ 1 (perf/array.jl:16 arrays) and Bool + Bool
    ints = rng.integers(-10, 11, (512, 1000), dtype=np.int64)
    assert np.array_equal(rk.Array(rk.materialize(L(rk.ROCArray(ints)) + 1)), ints + 1)
    m1, m2 = rng.random(1000) < 0.5, rng.random(1000) < 0.5
    got = rk.materialize(L(rk.ROCArray(m1)) + L(rk.ROCArray(m2)))
    assert got.dtype == np.int64 and np.array_equal(rk.Array(got), m1.astype(np.int64) + m2)
    # `/` and math functions of integers are Float64 in Julia
    got = rk.materialize(L(rk.ROCArray(ints)) / L(rk.ROCArray(ints + 20)))
    assert got.dtype == np.float64 and np.array_equal(rk.Array(got), ints / (ints + 20))
    got = rk.materialize(rk.broadcast.sqrt(L(rk.ROCArray(ints + 10))))
    assert got.dtype == np.float64
    np.testing.assert_allclose(rk.Array(got), np.sqrt(ints + 10), rtol=1e-15)
    # an Int64 program into an Int32 destination keeps the low bits; into a Float32 destination converts
    d32 = rk.ROCArray(dims=(100_003,), dtype=np.int32)
    rk.materialize_(d32, L(rk.ROCArray(a64)) + L(rk.ROCArray(b64)))
    with np.errstate(over="ignore"):
        assert np.array_equal(rk.Array(d32), (a64 + b64).astype(np.int32))
    small = rng.integers(-1000, 1000, 5000, dtype=np.int64)
    f32 = rk.ROCArray(dims=(5000,), dtype=np.float32)
    rk.materialize_(f32, L(rk.ROCArray(small)) * 2)
    assert np.array_equal(rk.Array(f32), (small * 2).astype(np.float32))
    # copies of Int64 beyond 2^53 are exact
    big = np.array([2**62 + 1, -(2**62) - 3, 2**53 + 1], dtype=np.int64)
    assert np.array_equal(rk.Array(rk.materialize(L(rk.ROCArray(big)))), big)


@pytest.mark.parametrize("dtype", [np.int8, np.int16, np.uint16, np.uint8])
def test_narrow_integer_arrays(rk, dtype):
    """Int8 / Int16 / UInt16 (and UInt8) operands and destinations: integer programs compute in Int64, the store keeps
    the low bits (Julia's wrap-around), and a narrow intermediate is wrapped before an order-sensitive operation."""
    rng = np.random.default_rng(60)
    L = rk.lazy
    info = np.iinfo(dtype)
    for shape in ((1000,), (300, 70), (257, 3, 5), (4096, 64)):
        a = rng.integers(info.min, info.max + 1, shape).astype(dtype)
        b = rng.integers(info.min, info.max + 1, shape).astype(dtype)
        da, db = rk.ROCArray(a), rk.ROCArray(b)
        with np.errstate(over="ignore"):
            got = rk.materialize(L(da) + L(db))
            assert got.dtype == dtype and np.array_equal(rk.Array(got), (a + b).astype(dtype))
            got = rk.materialize(L(da) * L(db) - L(da))
            assert got.dtype == dtype and np.array_equal(rk.Array(got), (a * b - a).astype(dtype))
            got = rk.materialize(rk.broadcast.max_(L(da), L(db)))
            assert got.dtype == dtype and np.array_equal(rk.Array(got), np.maximum(a, b))
            # the sum wraps in the narrow type before the comparison / max sees it
            got = rk.materialize(rk.broadcast.max_(L(da) + L(db), L(da)))
            assert got.dtype == dtype and np.array_equal(rk.Array(got), np.maximum((a + b).astype(dtype), a))
            got = rk.materialize((L(da) + L(db)) > L(da))
            assert got.dtype == np.bool_ and np.array_equal(rk.Array(got), (a + b).astype(dtype) > a)
        # mixed with a wider type: promotes; into a Float32 destination: converts
        w = rng.integers(-1000, 1000, shape).astype(np.int32)
        got = rk.materialize(L(da) + L(rk.ROCArray(w)))
        with np.errstate(over="ignore"):
            assert got.dtype == np.promote_types(dtype, np.int32) and np.array_equal(rk.Array(got), (a.astype(got.dtype) + w.astype(got.dtype)))
        f32 = rk.ROCArray(dims=shape, dtype=np.float32)
        rk.materialize_(f32, L(da) * 2)
        assert np.array_equal(rk.Array(f32), (a.astype(np.int64) * 2).astype(np.float32))      # Int8 * Int is an Int
        # a narrow destination of a wider program keeps the low bits
        dn = rk.ROCArray(dims=shape, dtype=dtype)
        rk.materialize_(dn, L(rk.ROCArray(w)) * 3)
        assert np.array_equal(rk.Array(dn), (w.astype(np.int64) * 3).astype(dtype))
    # a row vector against a matrix
    m = rng.integers(info.min, info.max + 1, (130, 50)).astype(dtype)
    r = rng.integers(info.min, info.max + 1, (1, 50)).astype(dtype)
    with np.errstate(over="ignore"):
        assert np.array_equal(rk.Array(rk.materialize(L(rk.ROCArray(m)) - L(rk.ROCArray(r)))), (m - r).astype(dtype))


def test_three_operand_trees_all_operator_pairs(rk):
    """(u op1 v) op2 w and u op1 (v op2 w) run on a fused evaluator: every operator pair, both shapes, repeated and
    scalar and extruded operands; Float32 results equal NumPy's un-fused Float32 arithmetic bit for bit."""
    rng = _rng(21)
    shape = (132, 77)
    x = (rng.random(shape, dtype=np.float32) + np.float32(0.5))
    y = (rng.random(shape, dtype=np.float32) + np.float32(0.5))
    col = (rng.random((132, 1), dtype=np.float32) + np.float32(0.5))
    row = (rng.random((1, 77), dtype=np.float32) + np.float32(0.5))
    X, Y, Cc, R = (rk.ROCArray(a) for a in (x, y, col, row))
    B = rk.broadcast
    ops = {"+": (lambda a, b: a + b, np.add), "-": (lambda a, b: a - b, np.subtract), "*": (lambda a, b: a * b, np.multiply),
           "/": (lambda a, b: a / b, np.divide), "max": (B.max_, np.maximum), "min": (B.min_, np.minimum)}
    two = np.float32(2)
    triples = [((X, x), (Y, y), (Cc, col)), ((X, x), (X, x), (Y, y)), ((two, two), (X, x), (R, row)), ((Cc, col), (R, row), (X, x))]
    lz = rk.lazy
    for (u, hu), (v, hv), (w, hw) in triples:
        for n1, (f1, g1) in ops.items():
            for n2, (f2, g2) in ops.items():
                got = rk.Array(rk.materialize(f2(f1(lz(u), lz(v)), lz(w))))
                np.testing.assert_array_equal(got, g2(g1(hu, hv), hw).astype(np.float32), err_msg=f"({n1}) {n2}")
                got = rk.Array(rk.materialize(f1(lz(u), f2(lz(v), lz(w)))))
                np.testing.assert_array_equal(got, g1(hu, g2(hv, hw)).astype(np.float32), err_msg=f"{n1} ({n2})")
    k = rng.integers(-2**31, 2**31, shape).astype(np.int32)
    j = rng.integers(-2**31, 2**31, shape).astype(np.int32)
    K, J = rk.ROCArray(k), rk.ROCArray(j)
    with np.errstate(over="ignore"):
        for n1 in ("+", "-", "*"):
            for n2 in ("+", "-", "*"):
                f1, g1 = ops[n1]
                f2, g2 = ops[n2]
                got = rk.materialize(f2(f1(lz(K), lz(J)), lz(K)))
                assert got.dtype == np.int32 and np.array_equal(rk.Array(got), g2(g1(k, j), k)), (n1, n2)


def test_left_deep_chains(rk):
    """((u0 op u1) op u2) ... up to eight operands run without a value stack; same bits as NumPy's Float32."""
    rng = _rng(22)
    shape = (260, 37)
    full = [rng.random(shape, dtype=np.float32) + np.float32(0.5) for _ in range(3)]
    col = rng.random((260, 1), dtype=np.float32) + np.float32(0.5)
    row = rng.random((1, 37), dtype=np.float32) + np.float32(0.5)
    row2 = rng.random((1, 37), dtype=np.float32) + np.float32(0.5)
    hosts = [full[0], row, row2, col, full[1], np.float32(1.5), full[2], full[0]]
    devs = [rk.ROCArray(h) if isinstance(h, np.ndarray) else h for h in hosts]
    lz = rk.lazy
    B = rk.broadcast
    gpu_ops = [lambda a, b: a - b, lambda a, b: a / b, lambda a, b: a * b, lambda a, b: a + b, B.max_, B.min_, lambda a, b: a - b]
    cpu_ops = [np.subtract, np.divide, np.multiply, np.add, np.maximum, np.minimum, np.subtract]
    for n in range(4, 9):                                     # 4 .. 8 operands (3 have their own evaluator)
        for shift in range(3):
            g, c = lz(devs[0]), hosts[0]
            for k in range(1, n):
                j = (k - 1 + shift) % len(gpu_ops)
                g = gpu_ops[j](g, lz(devs[k]))
                c = cpu_ops[j](c, hosts[k])
            np.testing.assert_array_equal(rk.Array(rk.materialize(g)), c.astype(np.float32), err_msg=f"{n} operands, shift {shift}")
    k = rng.integers(-2**31, 2**31, (4, 1000)).astype(np.int32)
    K = rk.ROCArray(k)
    with np.errstate(over="ignore"):
        got = rk.materialize(((lz(K) * lz(K) - lz(K)) * np.int32(3) + lz(K)) * lz(K))
        assert got.dtype == np.int32 and np.array_equal(rk.Array(got), ((k * k - k) * np.int32(3) + k) * k)


def test_float16_arrays(rk):
    """Float16 operands and destinations: Float32 arithmetic with a rounding to Float16 after every operation whose Julia
    type is Float16 -- what Julia (and NumPy) do -- so results are bit-identical to NumPy's Float16 arithmetic."""
    rng = _rng(23)
    shape = (130, 67)
    x = rng.standard_normal(shape).astype(np.float16)
    y = (rng.random(shape) + 0.5).astype(np.float16)
    col = rng.standard_normal((130, 1)).astype(np.float16)
    f = rng.standard_normal(shape).astype(np.float32)
    X, Y, Cc, F = (rk.ROCArray(a) for a in (x, y, col, f))
    lz = rk.lazy
    h = np.float16
    cases = [
        (lz(X) + lz(Y), x + y), (lz(X) * lz(Y) - lz(Cc), x * y - col), (lz(X) / lz(Y), x / y),
        ((lz(X) + lz(Y)) * (lz(X) - lz(Y)) / lz(Y), (x + y) * (x - y) / y),
        (h(1.5) * lz(X) + lz(Cc), h(1.5) * x + col), (rk.broadcast.abs2(lz(X)) + lz(Y), x * x + y),
        (rk.broadcast.max_(lz(X), lz(Cc)) - rk.broadcast.min_(lz(X), lz(Y)), np.maximum(x, col) - np.minimum(x, y)),
        (lz(X) + 2, x + h(2)),                                   # an Int literal keeps Float16
    ]
    for bc, want in cases:
        got = rk.materialize(bc)
        assert got.dtype == np.float16
        np.testing.assert_array_equal(rk.Array(got), want.astype(np.float16))
    got = rk.materialize(lz(X) * lz(F) + lz(Y))                  # Float16 with Float32: a Float32 program, nothing rounded
    assert got.dtype == np.float32
    np.testing.assert_array_equal(rk.Array(got), x.astype(np.float32) * f + y.astype(np.float32))
    got = rk.materialize((lz(X) + lz(Y)) * lz(F))                # the Float16 sum is rounded before it meets the Float32
    np.testing.assert_array_equal(rk.Array(got), (x + y).astype(np.float32) * f)
    dest = rk.ROCArray(dims=shape, dtype=np.float16)              # Float32 program into a Float16 destination
    rk.materialize_(dest, lz(F) * np.float32(0.5))
    np.testing.assert_array_equal(rk.Array(dest), (f * np.float32(0.5)).astype(np.float16))
    got = rk.materialize(rk.broadcast.exp(lz(X)))
    assert got.dtype == np.float16
    np.testing.assert_allclose(rk.Array(got).astype(np.float64), np.exp(x.astype(np.float64)), rtol=2.0**-10)
    assert np.array_equal(rk.Array(rk.materialize(lz(X) > lz(Y))), x > y)
    s = rk.sum(lambda v: v * v, X)                               # closures over Float16 arrays: map first, then reduce
    assert isinstance(s, np.float16) and abs(float(s) - float((x * x).astype(np.float64).sum())) <= 2.0**-9 * float((x * x).astype(np.float64).sum())


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16, np.int32, np.int16, np.int64])
@pytest.mark.parametrize("shape", [(1 << 16,), (4100,), (300, 64), (130, 67), (64, 1, 50)])
def test_one_and_two_operand_trees(rk, dtype, shape):
    """Programs of the form g2(g1(f0b(f0a(u)) op f1b(f1a(v)))) have an evaluator without a value stack; every form it takes is
    checked against NumPy evaluated operation by operation in the element type (Float16: rounded after every
    operation; integers: wrap-around), on flat, rows and indexed shapes."""
    rng = _rng(31)
    B = rk.broadcast
    lz = rk.lazy
    d = np.dtype(dtype)
    if d.kind == "f":
        x = (rng.standard_normal(shape) * 2).astype(dtype)
        y = (rng.random(shape) + 0.5).astype(dtype)
    else:
        x = rng.integers(-90, 90, shape).astype(dtype)
        y = rng.integers(1, 90, shape).astype(dtype)
    col = y[..., :1].copy()                      # extruded along the last dim
    X, Y, Cc = rk.ROCArray(x), rk.ROCArray(y), rk.ROCArray(col)
    T = dtype
    exact = [
        (-lz(X), -x), (B.abs_(lz(X)), np.abs(x)), (B.abs2(lz(X)), x * x), (lz(X) * lz(X), x * x), (lz(X) + lz(X), x + x),
        (-B.abs_(lz(X)), -np.abs(x)), (B.abs2(lz(X)) + B.abs2(lz(Y)), (x * x + y * y).astype(T)),
        (B.abs2(lz(X) - lz(Y)), ((x - y) * (x - y)).astype(T)), (-(lz(X) * lz(Cc)), -(x * col)),
        (B.abs_(lz(X)) - B.abs_(lz(Cc)), np.abs(x) - np.abs(col)), (B.max_(-lz(X), lz(Y)), np.maximum(-x, y)),
        (B.abs_(-B.abs2(lz(X))), np.abs(-(x * x))),
        # binary operators with a scalar count as unary functions of the tree: a .* x .+ b .* y, c .- abs.(x), 2 .* (x .+ y) .- 1
        (T(3) * lz(X) + T(2) * lz(Y), (T(3) * x + T(2) * y).astype(T)), (T(5) - B.abs_(lz(X)), (T(5) - np.abs(x)).astype(T)),
        (T(2) * (lz(X) + lz(Y)) - T(1), (T(2) * (x + y) - T(1)).astype(T)), (B.max_(lz(X) * T(2), T(1)) + lz(Cc), (np.maximum(x * T(2), T(1)) + col).astype(T)),
        (lz(X) ** 2, x * x), ((lz(X) - lz(Y)) ** 2, ((x - y) * (x - y)).astype(T)),
    ]
    if d.kind == "f":
        one = T(1)
        exact += [
            (B.sqrt(B.abs_(lz(X))), np.sqrt(np.abs(x))), (B.inv(lz(Y)), (one / y).astype(T)), (one / lz(Y), (one / y).astype(T)),
            (B.sqrt(lz(Y)) * B.sqrt(lz(Y)), (np.sqrt(y) * np.sqrt(y)).astype(T)), (B.sqrt(B.abs2(lz(X)) + B.abs2(lz(Y))), np.sqrt((x * x + y * y).astype(T))),
            (B.isnan(lz(X) / lz(X)), np.isnan(x / x)),
        ]
    # three operands: m(f(u) op f(v)) op f(w) on either side, the same array in several places, three scalars
    z = x[..., ::-1].copy() if x.ndim > 1 else x[::-1].copy()
    Z = rk.ROCArray(z)
    exact += [
        (lz(X) * lz(Y) + B.abs_(lz(Z)), (x * y + np.abs(z)).astype(T)), (B.abs_(lz(Z)) - lz(X) * lz(Y), (np.abs(z) - x * y).astype(T)),
        (T(2) * lz(X) + T(3) * lz(Y) + T(5) * lz(Z), (T(2) * x + T(3) * y + T(5) * z).astype(T)),
        (B.abs2(lz(X)) + B.abs2(lz(Y)) + B.abs2(lz(Z)), (x * x + y * y + z * z).astype(T)),
        (-(lz(X) - lz(Y)) * (lz(X) + T(1)), (-(x - y) * (x + T(1))).astype(T)), ((lz(X) + lz(Z)) * lz(Z) - lz(X), ((x + z) * z - x).astype(T)),
        (B.max_(lz(X), lz(Y)) - B.min_(lz(Z), lz(X)), np.maximum(x, y) - np.minimum(z, x)),
        (lz(X) * lz(Cc) + lz(Z), (x * col + z).astype(T)),                       # an extruded operand: rows mode, the interpreter's
    ]
    # muladd(p, q, r) = p * q + r, one rounding at the end for Float16 (computed in Float32)
    wide = np.float32 if dtype == np.float16 else dtype
    exact += [(B.muladd(lz(X), lz(Y), lz(Z)), (x.astype(wide) * y.astype(wide) + z.astype(wide)).astype(T)),
              (B.muladd(lz(X), lz(X), lz(Cc)), (x.astype(wide) * x.astype(wide) + col.astype(wide)).astype(T))]
    if d.kind == "f":
        exact += [((lz(X) - lz(Z)) / B.sqrt(lz(Y) + T(0.5)), ((x - z) / np.sqrt(y + T(0.5))).astype(T))]
    for bc, want in exact:
        got = rk.materialize(bc)
        np.testing.assert_array_equal(rk.Array(got), np.asarray(want).astype(got.dtype))
    if d.kind == "f":
        # transcendental functions: the device routines are within an ulp or two of the correctly rounded value
        tol = {2: 2.0**-9, 4: 4e-7, 8: 1e-15}[d.itemsize]
        x64, y64 = x.astype(np.float64), y.astype(np.float64)
        close = [
            (B.exp(lz(X)), np.exp(x64)), (B.tanh(lz(X)), np.tanh(x64)), (B.log(lz(Y)), np.log(y64)), (B.sin(lz(X)) * B.cos(lz(Y)), np.sin(x64) * np.cos(y64)),
            (T(1) / (T(1) + B.exp(-lz(X))), 1 / (1 + np.exp(-x64))), (B.exp(-B.abs2(lz(X))), np.exp(-x64 * x64)), (B.log(B.exp(lz(X)) + T(1)), np.log(np.exp(x64) + 1)),
            (lz(X) * lz(Y) + B.sin(lz(Z)), x64 * y64 + np.sin(z.astype(np.float64))), (B.exp(lz(X) - lz(Y)) * lz(Z), np.exp(x64 - y64) * z.astype(np.float64)),
        ]
        for bc, want in close:
            got = rk.Array(rk.materialize(bc)).astype(np.float64)
            np.testing.assert_allclose(got, want, rtol=4 * tol, atol=4 * tol)


@pytest.mark.parametrize("shape", [(1 << 16,), (4100,), (4096 + 8,), (256, 96), (130, 67)])
def test_narrow_arrays_in_the_fused_evaluators(rk, shape):
    """Float16 programs whose every operation rounds run in the fused evaluators (the rounding tokens become a rounding of
    every intermediate), eight elements a lane where sizes and alignment allow; comparisons and logic of two arrays too.
    Bit-identical to NumPy's Float16 arithmetic, whichever kernel a shape selects."""
    rng = _rng(29)
    h = np.float16
    x = rng.standard_normal(shape).astype(h)
    y = (rng.random(shape) + 0.5).astype(h)
    w = (rng.standard_normal(shape) * 0.5).astype(h)
    g = (rng.random(shape) + 1.0).astype(h)
    X, Y, W, G = (rk.ROCArray(a) for a in (x, y, w, g))
    lz = rk.lazy
    cases = [
        (lz(X) + lz(Y), x + y), (lz(X) - lz(Y), x - y), (lz(X) * lz(Y), x * y), (lz(X) / lz(Y), x / y),
        (rk.broadcast.max_(lz(X), lz(Y)), np.maximum(x, y)),
        (h(1.5) * lz(X) + lz(Y), h(1.5) * x + y),                          # (u op v) op w
        (lz(X) + lz(Y) * lz(W), x + y * w),                                # u op (v op w)
        ((lz(X) - lz(W)) / lz(Y) * lz(G) + lz(W), (x - w) / y * g + w),      # a left chain of five operands
    ]
    for bc, want in cases:
        got = rk.materialize(bc)
        assert got.dtype == h
        np.testing.assert_array_equal(rk.Array(got), want.astype(h))
    got = rk.Array(rk.materialize(h(0.5) * lz(X) + lz(Y) * rk.broadcast.exp(lz(W))))
    e = np.exp(w.astype(np.float32)).astype(h)                             # exp itself within an ulp of Float16; the rest exact
    lo = h(0.5) * x + y * np.nextafter(e, h(-np.inf)); hi = h(0.5) * x + y * np.nextafter(e, h(np.inf))
    assert np.all((got >= np.minimum(lo, hi)) & (got <= np.maximum(lo, hi)))
    # Bool results of comparisons, logic of Bool arrays, Int16 arithmetic and order
    a = rng.integers(-300, 300, shape).astype(np.int16)
    b = rng.integers(-300, 300, shape).astype(np.int16)
    p = rng.random(shape) < 0.5
    q = rng.random(shape) < 0.5
    A, B, P, Q = (rk.ROCArray(v) for v in (a, b, p, q))
    for bc, want in [(lz(X) > lz(Y), x > y), (lz(X) <= lz(W), x <= w), (lz(A) < lz(B), a < b), (lz(A) == lz(B), a == b), (lz(A) != lz(B), a != b),
                     (lz(P) & lz(Q), p & q), (lz(P) | lz(Q), p | q), (lz(A) >= lz(B), a >= b)]:
        got = rk.materialize(bc)
        assert got.dtype == np.bool_
        np.testing.assert_array_equal(rk.Array(got), want)
    for bc, want in [(lz(A) + lz(B), a + b), (lz(A) * lz(B), a * b), (rk.broadcast.min_(lz(A), lz(B)), np.minimum(a, b)), (lz(A) - lz(B) * lz(A), a - b * a)]:
        got = rk.materialize(bc)
        assert got.dtype == np.int16
        np.testing.assert_array_equal(rk.Array(got), want.astype(np.int16))


@pytest.mark.parametrize("shape,others", [((3, 40_000), [(3, 1), (1, 40_000)]), ((17, 4000), [(17, 1), (1, 4000)]), ((5, 7, 800), [(5, 1, 800), (1, 7, 1)]),
                                          ((2, 2, 2, 30_000), [(2, 1, 2, 1), (1, 2, 1, 30_000)]), ((6, 10_002), [(1, 10_002), (6, 10_002)]),
                                          ((63, 4, 100), [(63, 1, 100), (1, 4, 1)]), ((3, 40_001), [(1, 40_001), (3, 1)]), ((17, 4001), [(17, 1), (1, 4001)]),
                                          ((5, 3, 333), [(1, 3, 333), (5, 1, 1)]), ((3, 3, 3, 3, 1000), [(3, 1, 3, 1, 1000), (1, 3, 1, 3, 1)])])
def test_short_odd_first_dim(rk, shape, others):
    """A dense destination whose dim 0 is short and no whole number of 16-byte vectors (3 x N .+ 1 x N): threads along
    the linear index, extruded operands gathered; totals that are no multiple of 4 end in a partial vector.  Float32, mixed element types (Float64 and Int32 operands into a
    Float32 / Float64 destination), an integer program, a deep tree (the interpreter), and five merged dims (lanes
    along dim 0 again)."""
    rng = np.random.default_rng(211)
    L = rk.lazy
    A = rng.standard_normal(shape).astype(np.float32)
    u = rng.standard_normal(others[0]).astype(np.float32)
    v = rng.standard_normal(others[1]).astype(np.float32)
    dA, du, dv = rk.ROCArray(A), rk.ROCArray(u), rk.ROCArray(v)
    np.testing.assert_array_equal(rk.Array(rk.materialize(L(dA) + L(du))), A + u)
    np.testing.assert_array_equal(rk.Array(rk.materialize((L(dA) - L(du)) * L(dv))), (A - u) * v)
    np.testing.assert_array_equal(rk.Array(rk.materialize(L(du) * L(dv))), (u * v).astype(np.float32) + np.zeros(shape, np.float32))
    deep = rk.materialize(rk.broadcast.max_(L(dA) * L(du) + L(dv), L(dA) - np.float32(0.25)) * (L(du) + L(dv)) - L(dA) * L(dA))
    np.testing.assert_array_equal(rk.Array(deep), np.maximum(A * u + v, A - np.float32(0.25)) * (u + v) - A * A)
    u64 = rng.standard_normal(others[0])
    np.testing.assert_array_equal(rk.Array(rk.materialize(L(dA) + L(rk.ROCArray(u64)))), A + u64)             # Float64 result
    iA = rng.integers(-1000, 1000, shape).astype(np.int32)
    iu = rng.integers(-1000, 1000, others[0]).astype(np.int32)
    got = rk.Array(rk.materialize(L(rk.ROCArray(iA)) * L(rk.ROCArray(iu)) - L(rk.ROCArray(iA))))
    assert got.dtype == np.int32 and np.array_equal(got, iA * iu - iA)
    dest = rk.ROCArray(dims=shape, dtype=np.float32)                                                            # in place: dest is an operand
    rk.materialize_(dest, L(dA) + np.float32(0))
    rk.materialize_(dest, L(dest) * L(dv) + L(du))
    np.testing.assert_array_equal(rk.Array(dest), A * v + u)
