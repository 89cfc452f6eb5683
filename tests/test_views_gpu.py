"""Broadcast with wrapper operands and destinations -- views, transposes, PermutedDimsArrays (the reference's
ROCArrayStyle covers "any ROCArray or wrapper", src/broadcast.jl:7-10) -- against NumPy slicing, through the C ABI.
`+ - *` results are bit-exact (same Float32 operations in the same order)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _f32(rng, shape):
    return rng.standard_normal(shape).astype(np.float32)


def test_view_operands(rk):
    rng = np.random.default_rng(1)
    A = _f32(rng, (40, 30)); B = _f32(rng, (40, 30)); v = _f32(rng, 40)
    dA, dB, dv = rk.ROCArray(A), rk.ROCArray(B), rk.ROCArray(v)
    L = rk.lazy
    # rows 3:22, columns 2:2:30 of A plus a dense block
    got = rk.Array(rk.materialize(L(rk.view(dA, (3, 22), (2, 2, 30))) + L(rk.ROCArray(np.ascontiguousarray(B[2:22, 1:30:2])))))
    assert np.array_equal(got, A[2:22, 1:30:2] + B[2:22, 1:30:2])
    # a column view and a reversed row range
    got = rk.Array(rk.materialize(L(rk.view(dA, None, 7)) * L(dv)))
    assert np.array_equal(got, A[:, 6] * v)
    got = rk.Array(rk.materialize(L(rk.view(dA, (40, -1, 1), None)) - L(dB)))
    assert np.array_equal(got, A[::-1, :] - B)
    # a row view (stride 40 along its only dim)
    got = rk.Array(rk.materialize(np.float32(2) * L(rk.view(dA, 5, None))))
    assert np.array_equal(got, np.float32(2) * A[4, :])
    assert np.array_equal(rk.Array(rk.view(dA, (2, 39), (1, 30))), A[1:39, :])


def test_transpose_and_permuteddims_operands(rk):
    rng = np.random.default_rng(2)
    A = _f32(rng, (64, 48)); B = _f32(rng, (48, 64)); T3 = _f32(rng, (8, 12, 20))
    L = rk.lazy
    got = rk.Array(rk.materialize(L(rk.transpose(rk.ROCArray(A))) + L(rk.ROCArray(B))))
    assert np.array_equal(got, A.T + B)
    v = _f32(rng, 48)
    got = rk.Array(rk.materialize(L(rk.ROCArray(A)) * L(rk.transpose(rk.ROCArray(v)))))       # 64x48 .* 1x48
    assert np.array_equal(got, A * v[None, :])
    P = rk.PermutedDimsArray(rk.ROCArray(T3), (3, 1, 2))
    assert P.dims == (20, 8, 12)
    assert np.array_equal(rk.Array(P), np.transpose(T3, (2, 0, 1)))
    assert np.array_equal(rk.Array(rk.materialize(L(P) * np.float32(3))), np.transpose(T3, (2, 0, 1)) * np.float32(3))
    # against the dense permutedims kernel
    assert np.array_equal(rk.Array(P), rk.Array(rk.permutedims(rk.ROCArray(T3), (3, 1, 2))))


def test_view_destinations(rk):
    rng = np.random.default_rng(3)
    C = _f32(rng, (50, 37)); X = _f32(rng, (20, 37)); Y = _f32(rng, (37, 50))
    L = rk.lazy
    dC = rk.ROCArray(C)
    rk.materialize_(rk.view(dC, (11, 30), None), L(rk.ROCArray(X)) * np.float32(2))            # @view(C[11:30, :]) .= 2X
    want = C.copy(); want[10:30, :] = X * np.float32(2)
    assert np.array_equal(rk.Array(dC), want)
    rk.materialize_(rk.transpose(dC), L(rk.ROCArray(Y)) + np.float32(1))                        # transpose(C) .= Y .+ 1
    assert np.array_equal(rk.Array(dC), (Y + np.float32(1)).T)
    rk.fill_(rk.view(dC, (1, 2, 49), (37, -3, 1)), 7.0)                                          # C[1:2:49, 37:-3:1] .= 7
    want = (Y + np.float32(1)).T.copy(); want[0:49:2, 36::-3] = 7.0
    assert np.array_equal(rk.Array(dC), want)
    # in-place update of a view from itself and a row vector: v .= v .+ r
    r = _f32(rng, 37)
    vw = rk.view(dC, (5, 44), None)
    rk.materialize_(vw, L(vw) + L(rk.transpose(rk.ROCArray(r))))
    want[4:44, :] = want[4:44, :] + r[None, :]
    assert np.array_equal(rk.Array(dC), want)


def test_large_strided_shapes_and_vector_path(rk):
    rng = np.random.default_rng(4)
    A = _f32(rng, (1024, 513))
    dA = rk.ROCArray(A)
    L = rk.lazy
    # aligned row range with whole 16-byte vectors: the vector lanes stay on
    got = rk.Array(rk.materialize(L(rk.view(dA, (257, 768), (2, 512))) * np.float32(0.5)))
    assert np.array_equal(got, A[256:768, 1:512] * np.float32(0.5))
    # unaligned start, odd extents
    got = rk.Array(rk.materialize(L(rk.view(dA, (2, 1000), (3, 511))) + L(rk.view(dA, (3, 1001), (1, 509)))))
    assert np.array_equal(got, A[1:1000, 2:511] + A[2:1001, 0:509])
    # matrix transpose through the broadcast kernel equals the tiled transpose
    assert np.array_equal(rk.Array(rk.transpose(dA)), A.T)


def test_views_are_refused_by_dense_ops(rk):
    d = rk.ROCArray(np.arange(12, dtype=np.float32).reshape(3, 4))
    with pytest.raises(rk.UnsupportedError):
        rk.sum(rk.view(d, (1, 2), None))
    with pytest.raises(IndexError):
        rk.view(d, (1, 5), None)
    with pytest.raises(IndexError):
        rk.view(d, 4, None)


def test_operands_that_alias_the_destination_are_copied_first(rk):
    """``Broadcast.broadcast_unalias``: the right-hand side is evaluated as if no element had been written yet."""
    rng = np.random.default_rng(31)
    a = rng.standard_normal((300, 257)).astype(np.float32)
    A = rk.ROCArray(a)
    rk.materialize_(rk.view(A, (1, 299), None), rk.lazy(rk.view(A, (2, 300), None)) + np.float32(1))     # rows move up by one
    want = a.copy()
    want[0:299, :] = a[1:300, :] + np.float32(1)
    assert np.array_equal(rk.Array(A), want)
    s = rng.standard_normal((129, 129)).astype(np.float32)
    S = rk.ROCArray(s)
    rk.materialize_(S, rk.lazy(rk.transpose(S)) * np.float32(2))                                       # S .= 2 .* transpose(S)
    assert np.array_equal(rk.Array(S), s.T * np.float32(2))
    x = rng.standard_normal(10_001).astype(np.float32)
    X = rk.ROCArray(x)
    rk.materialize_(X, rk.lazy(X) * rk.lazy(X) + np.float32(1))                                         # the same elements in place
    assert np.array_equal(rk.Array(X), x * x + np.float32(1))
    rk.materialize_(rk.view(X, (1, 5000)), rk.lazy(rk.view(X, (5001, -1, 2))))                          # reversed overlapping range
    want = x * x + np.float32(1)
    want[0:5000] = want[1:5001][::-1].copy()
    assert np.array_equal(rk.Array(X), want)
    from amdgpu_jl_amd.broadcast import plan_materialize
    with pytest.raises(rk.UnsupportedError):
        plan_materialize(rk.view(A, (1, 299), None), rk.lazy(rk.view(A, (2, 300), None)))


# ---- wrapper arrays in reductions and scans (rk_mapreduce_strided / rk_accumulate_strided) -----------------------------
def test_mapreducedim_into_a_transpose_returns_it(rk):
    # test/core/rocarray_base.jl:263-267: mapreducedim!(identity, +, transpose(zeros(2, 3)), rand(3, 2, 10)) === R
    a = np.random.default_rng(41).random((3, 2, 10), dtype=np.float32)
    P = rk.zeros(np.float32, 2, 3)
    R = rk.transpose(P)
    assert R.dims == (3, 2)
    out = rk.mapreducedim_(rk.identity, rk.add, R, rk.ROCArray(a))
    assert out is R
    np.testing.assert_allclose(rk.Array(P), a.astype(np.float64).sum(axis=2).T, rtol=1e-5)       # parent[j, i] = sum_k A[i, j, k]
    np.testing.assert_allclose(rk.Array(R), a.astype(np.float64).sum(axis=2), rtol=1e-5)


@pytest.mark.parametrize("perm", [(2, 1, 3), (3, 1, 2), (3, 2, 1), (1, 3, 2)])
@pytest.mark.parametrize("dtype", [np.float32, np.int32])
def test_reductions_of_permuted_arrays(rk, perm, dtype):
    rng = np.random.default_rng(sum(perm) * 7 + 1)
    b = (rng.standard_normal((37, 50, 23)) * 100).astype(dtype)
    B = rk.ROCArray(b)
    A = rk.PermutedDimsArray(B, perm)                       # logical array = permutedims(b, perm)
    h = np.transpose(b, [p - 1 for p in perm])
    assert A.dims == h.shape
    for dims in (1, 2, 3, (1, 2), (1, 3), (1, 2, 3)):
        dd = (dims,) if isinstance(dims, int) else dims
        rshape = tuple(1 if (k + 1) in dd else n for k, n in enumerate(h.shape))
        out_dt = np.int64 if dtype == np.int32 else dtype
        R = rk.ROCArray(dims=rshape, dtype=out_dt)
        rk.mapreducedim_(rk.identity, rk.add, R, A)
        want = h.astype(np.float64 if dtype == np.float32 else np.int64).sum(axis=tuple(k - 1 for k in dd), keepdims=True)
        if dtype == np.float32:
            np.testing.assert_allclose(rk.Array(R), want, rtol=1e-5, atol=1e-2)
        else:
            assert np.array_equal(rk.Array(R), want)
        M = rk.ROCArray(dims=rshape, dtype=dtype)
        rk.mapreducedim_(rk.identity, rk.max_, M, A)
        assert np.array_equal(rk.Array(M), h.max(axis=tuple(k - 1 for k in dd), keepdims=True))
    # a permuted destination as well
    Rp = rk.zeros(np.int64 if dtype == np.int32 else dtype, h.shape[1], h.shape[0])
    rk.mapreducedim_(rk.identity, rk.add, rk.ROCView(Rp, 0, (h.shape[0], h.shape[1], 1), (h.shape[1], 1, 0)), A)
    want = h.astype(np.float64 if dtype == np.float32 else np.int64).sum(axis=2)
    if dtype == np.float32:
        np.testing.assert_allclose(rk.Array(Rp), want.T, rtol=1e-5, atol=1e-2)
    else:
        assert np.array_equal(rk.Array(Rp), want.T)


def test_views_with_gaps_are_not_native_in_reductions(rk):
    A = rk.ROCArray(np.ones((40, 30), dtype=np.float32))
    R = rk.zeros(np.float32, 1, 30)
    with pytest.raises(rk.UnsupportedError):
        rk.mapreducedim_(rk.identity, rk.add, R, rk.view(A, (1, 20), None))          # rows 1:20 of 40: gaps between the columns
    R2 = rk.zeros(np.float32, 40, 1)
    rk.mapreducedim_(rk.identity, rk.add, R2, rk.view(A, None, (11, 30)))             # whole columns: dense
    assert np.array_equal(rk.Array(R2), np.full((40, 1), 20, dtype=np.float32))


@pytest.mark.parametrize("dims", [1, 2])
def test_accumulate_on_transposes(rk, orc, dims):
    rng = np.random.default_rng(43 + dims)
    a = rng.integers(-1000, 1001, (300, 517), dtype=np.int32)
    A, B = rk.ROCArray(a), rk.zeros(np.int32, 300, 517)
    out = rk.accumulate_("add", rk.transpose(B), rk.transpose(A), dims=dims)
    assert out.dims == (517, 300)
    assert np.array_equal(rk.Array(B).T, orc.accumulate("add", np.ascontiguousarray(a.T), dims=dims))
    with pytest.raises(rk.UnsupportedError):
        rk.accumulate_("add", rk.zeros(np.int32, 517, 300), rk.transpose(A), dims=dims)      # laid out differently


def test_findmax_on_wrappers(rk, orc):
    """findmax / findmin(transpose(A); dims), (PermutedDimsArray(A, p); dims): the index comes back in the wrapper's
    coordinates and the first of equal winners is the first in the WRAPPER's column-major order -- checked against the
    oracle on the materialised wrapper, with planted ties, NaNs and signed zeros.  Orders of dims for which the parent's
    memory order would pick another winner or lay the outputs out otherwise are declined, not answered."""
    rng = np.random.default_rng(61)
    A = rng.integers(-3, 4, (300, 257)).astype(np.float32)                  # few distinct values: ties everywhere
    A[5, 7] = np.nan; A[5, 200] = np.nan; A[17, :] = 0.0; A[17, 3] = -0.0
    dA = rk.ROCArray(A)
    At = np.ascontiguousarray(A.T)

    def check(wrapper, host, dims):
        for gpu, cpu in ((rk.findmax, orc.findmax), (rk.findmin, orc.findmin)):
            gv, gi = gpu(wrapper, dims=dims)
            ov, oi = cpu(host, dims=dims)
            assert np.array_equal(rk.Array(gv), ov, equal_nan=True)
            assert np.array_equal(np.signbit(rk.Array(gv)), np.signbit(ov))
            assert np.array_equal(np.moveaxis(rk.Array(gi), 0, -1), oi)

    for dims in (1, 2):
        check(rk.transpose(dA), At, dims)
    with pytest.raises(NotImplementedError):
        rk.findmax(rk.transpose(dA))                                         # dims = : walks the reduced dims in another order
    T3 = rng.integers(-2, 3, (20, 33, 65)).astype(np.float64)
    d3 = rk.ROCArray(T3)
    for perm in ((2, 1, 3), (3, 1, 2), (1, 3, 2), (3, 2, 1), (2, 3, 1)):
        P = rk.PermutedDimsArray(d3, perm)
        host = np.ascontiguousarray(np.transpose(T3, tuple(p - 1 for p in perm)))
        served = 0
        for dims in (1, 2, 3, (1, 2), (2, 3), (1, 3)):
            try:
                check(P, host, dims)
                served += 1
            except NotImplementedError:
                pass                                                         # declined: the binding copies the wrapper first
        assert (served > 0) == (perm != (3, 2, 1))                           # a full reversal keeps no pair of dims in order
    ints = rng.integers(-5, 6, (129, 70)).astype(np.int32)
    for dims in (1, 2):
        for gpu, cpu in ((rk.findmax, orc.findmax), (rk.findmin, orc.findmin)):
            gv, gi = gpu(rk.transpose(rk.ROCArray(ints)), dims=dims)
            ov, oi = cpu(np.ascontiguousarray(ints.T), dims=dims)
            assert np.array_equal(rk.Array(gv), ov) and np.array_equal(np.moveaxis(rk.Array(gi), 0, -1), oi)
