"""GPU parity of permutedims / permutedims! against the oracle (NumPy transpose, pinned element by element in
tests/test_oracle.py), through the C ABI, bit-exact.  Shapes of perf/array.jl:151-155 first; the reference
repository has no test of its own for this op (it lives in GPUArrays)."""
import itertools

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _rand(rng, dtype, shape):
    dt = np.dtype(dtype)
    if dt.kind == "c":
        return (rng.random(shape) + 1j * rng.random(shape)).astype(dt)
    if dt.kind == "f":
        return rng.random(shape).astype(dt)
    if dt.kind == "b":
        return rng.random(shape) < 0.5
    return rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, shape, dtype=dt)


def _check(rk, orc, x, perm):
    got = rk.Array(rk.permutedims(rk.ROCArray(x), perm))
    want = orc.permutedims(x, perm)
    assert got.shape == want.shape and got.dtype == want.dtype
    assert np.array_equal(got.view(np.uint8), np.ascontiguousarray(want).view(np.uint8))


@pytest.mark.parametrize("shape,perm", [((512, 1000), (2, 1)), ((512, 40, 25), (3, 1, 2)), ((512, 10, 10, 10), (2, 1, 4, 3))])
@pytest.mark.parametrize("dtype", [np.float32, np.int64])
def test_perf_suite_shapes(rk, orc, shape, perm, dtype):
    _check(rk, orc, _rand(np.random.default_rng(1), dtype, shape), perm)


@pytest.mark.parametrize("perm", list(itertools.permutations((1, 2, 3))))
@pytest.mark.parametrize("shape", [(5, 7, 3), (64, 65, 2), (100, 1, 37), (1, 129, 66), (130, 67, 1)])
def test_all_3d_permutations(rk, orc, perm, shape):
    _check(rk, orc, _rand(np.random.default_rng(2), np.float32, shape), perm)


@pytest.mark.parametrize("dtype", [np.bool_, np.int16, np.float16, np.float32, np.float64, np.complex128])
@pytest.mark.parametrize("shape,perm", [((1000, 513), (2, 1)), ((33, 4, 65), (3, 2, 1)), ((16, 8, 9), (1, 3, 2)), ((70, 3, 5, 4), (4, 1, 3, 2))])
def test_element_sizes(rk, orc, dtype, shape, perm):
    _check(rk, orc, _rand(np.random.default_rng(3), dtype, shape), perm)


def test_higher_ranks_merging_and_identity(rk, orc):
    rng = np.random.default_rng(4)
    x = _rand(rng, np.int32, (4, 3, 5, 2, 6, 3))
    for perm in [(1, 2, 3, 4, 5, 6), (3, 4, 1, 2, 5, 6), (5, 6, 1, 2, 3, 4), (6, 5, 4, 3, 2, 1), (2, 3, 1, 6, 4, 5), (1, 2, 5, 6, 3, 4)]:
        _check(rk, orc, x, perm)
    _check(rk, orc, _rand(rng, np.float32, (4096, 2048)), (2, 1))
    _check(rk, orc, _rand(rng, np.float32, (3, 100_000)), (2, 1))
    _check(rk, orc, _rand(rng, np.float32, (100_000, 3)), (2, 1))
    _check(rk, orc, _rand(rng, np.float32, (17,)), (1,))


def test_front_end(rk, orc):
    m = _rand(np.random.default_rng(5), np.float32, (6, 9))
    d = rk.ROCArray(m)
    assert np.array_equal(rk.Array(rk.permutedims(d)), m.T)
    v = rk.ROCArray(m[:, 0].copy())
    assert rk.permutedims(v).dims == (1, 6)
    dest = rk.ROCArray(dims=(9, 6), dtype=np.float32)
    assert rk.permutedims_(dest, d, (2, 1)) is dest
    with pytest.raises(ValueError):
        rk.permutedims(d, (1, 1))
    with pytest.raises(rk.DimensionMismatch):
        rk.permutedims_(rk.ROCArray(dims=(6, 9), dtype=np.float32), d, (2, 1))


@pytest.mark.parametrize("dtype", [np.bool_, np.int16, np.float32, np.float64, np.complex128])
@pytest.mark.parametrize("shape,perm", [((100_003, 3), (2, 1)), ((3, 100_003), (2, 1)), ((65_537, 4), (2, 1)), ((4, 65_537), (2, 1)),
                                        ((8, 8, 5000), (2, 1, 3)), ((2, 7, 3001), (2, 1, 3)), ((1000, 5, 7, 3), (2, 1, 4, 3)),
                                        ((6, 1000, 4), (3, 2, 1)), ((1, 5, 4099), (3, 2, 1)), ((8, 257, 2, 9), (3, 1, 4, 2)), ((2, 2, 2, 2, 70_001), (4, 3, 2, 1, 5)),
                                        ((2, 3, 100_001), (3, 2, 1)), ((100_001, 3, 2), (3, 2, 1)), ((2, 2, 2, 50_001, 3), (4, 3, 2, 1, 5)), ((4, 2, 70_001), (3, 1, 2))])
def test_short_contiguous_dims(rk, orc, dtype, shape, perm):
    """A short contiguous dim on either side (arrays of structures <-> structures of arrays, batches of tiny matrices)."""
    _check(rk, orc, _rand(np.random.default_rng(71), dtype, shape), perm)


@pytest.mark.parametrize("dtype", [np.bool_, np.int16, np.float32, np.float64, np.complex128])
@pytest.mark.parametrize("shape,perm", [((2, 100_001, 2), (3, 2, 1)), ((8, 5000, 8), (3, 2, 1)), ((4, 32, 3001), (3, 2, 1)), ((3001, 32, 4), (3, 2, 1)),
                                        ((17, 33, 65), (3, 2, 1)), ((3, 700, 5, 31), (4, 2, 3, 1)), ((31, 9, 1000), (3, 2, 1)), ((1000, 9, 31), (3, 2, 1)),
                                        ((5, 40, 6, 300), (3, 4, 2, 1)), ((16, 2, 3, 4, 500), (5, 2, 4, 3, 1)), ((12, 1025, 20), (3, 2, 1)), ((2, 3, 4, 5, 6, 700), (6, 5, 4, 3, 2, 1)),
                                        ((17, 20_001), (2, 1)), ((20_001, 17), (2, 1)), ((31, 5000), (2, 1)), ((9, 70_000), (2, 1)), ((70_000, 9), (2, 1)), ((12, 7, 3000), (3, 1, 2))])
def test_short_first_dims_with_a_third_dim(rk, orc, dtype, shape, perm):
    """The source's or the destination's first dim is short and neither side is a run of at most 8 elements: boxes of
    three dims through LDS ((2, N, 2) with perm (3, 2, 1): a tile per 4 elements otherwise)."""
    _check(rk, orc, _rand(np.random.default_rng(73), dtype, shape), perm)


@pytest.mark.parametrize("shape,perm,dtype", [((100, 100, 300), (2, 1, 3), np.float32), ((101, 99, 257), (2, 1, 3), np.int32),
                                              ((70, 80, 256), (2, 1, 3), np.float64), ((96, 72, 4, 70), (2, 1, 3, 4), np.float32),
                                              ((65, 110, 260), (2, 1, 3), np.uint32), ((77, 79, 300), (2, 1, 3), np.int64),
                                              ((5001, 601), (2, 1), np.float32), ((4097, 130), (2, 1), np.float64)])
def test_batches_of_small_matrices_and_odd_extents(rk, orc, shape, perm, dtype):
    """permutedims(A, (2, 1, 3)) of >= 256 matrices that 64 x 64 tiles would fill poorly: whole matrices through LDS
    (100 x 100 x 3000 Float32: 2.5 -> 5.5 TB/s).  The last two: a plain transpose whose extents are no whole vectors
    (the vector tiles with element-aligned accesses, tile columns dealt to the XCDs)."""
    _check(rk, orc, _rand(np.random.default_rng(5), dtype, shape), perm)
