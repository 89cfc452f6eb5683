"""GPU parity of reverse / reverse! (src/kernels/reverse.jl) against the oracle, through the C ABI; the cases of
test/hip_rocarray/reverse.jl:5-51 plus sizes that reach the 16-byte-unit path, all bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _rand(rng, dtype, shape):
    dt = np.dtype(dtype)
    if dt.kind == "f":
        return rng.random(shape).astype(dt)
    if dt.kind == "c":
        return (rng.random(shape) + 1j * rng.random(shape)).astype(dt)
    if dt.kind == "b":
        return rng.random(shape) < 0.5
    info = np.iinfo(dt)
    return rng.integers(info.min, info.max, shape, dtype=dt)


def _same(a, b):
    assert a.dtype == b.dtype and a.shape == b.shape
    assert np.array_equal(a.view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64])
@pytest.mark.parametrize("sz", [1, 2, 3, 4, 16, 128, 1024, 1025])
def test_1d_full_reverse(rk, orc, dtype, sz):
    # test/hip_rocarray/reverse.jl:6-16
    x = _rand(np.random.default_rng(sz), dtype, sz)
    xd = rk.ROCArray(x)
    _same(rk.Array(rk.reverse(xd)), orc.reverse(x))
    assert rk.reverse_(xd) is xd
    _same(rk.Array(xd), orc.reverse(x))


@pytest.mark.parametrize("offset", [1, 2, 13, 16])
def test_1d_partial(rk, orc, offset):
    # test/hip_rocarray/reverse.jl:19-30
    x = _rand(np.random.default_rng(offset), np.int16, 127)
    xd = rk.ROCArray(x)
    want = orc.reverse(x, offset, 127 - offset)
    _same(rk.Array(rk.reverse(xd, offset, 127 - offset)), want)
    rk.reverse_(xd, offset, 127 - offset)
    _same(rk.Array(xd), want)


@pytest.mark.parametrize("sz", [(1, 1), (1, 3), (4, 4), (127, 128), (1024, 1025)])
@pytest.mark.parametrize("dims", [None, 1, 2])
def test_2d(rk, orc, sz, dims):
    # test/hip_rocarray/reverse.jl:33-42
    x = _rand(np.random.default_rng(3), np.int16, sz)
    xd = rk.ROCArray(x)
    want = orc.reverse(x, dims=dims)
    _same(rk.Array(rk.reverse(xd, dims=dims)), want)
    _same(rk.Array(rk.reverse_(xd, dims=dims)), want)


def test_5d_dims_tuple(rk, orc):
    # test/hip_rocarray/reverse.jl:44-50
    x = _rand(np.random.default_rng(4), np.int16, (8, 9, 10, 11, 12))
    xd = rk.ROCArray(x)
    want = orc.reverse(x, dims=(1, 2, 4, 5))
    _same(rk.Array(rk.reverse(xd, dims=(1, 2, 4, 5))), want)
    _same(rk.Array(rk.reverse_(xd, dims=(1, 2, 4, 5))), want)


@pytest.mark.parametrize("dtype", [np.bool_, np.int16, np.float32, np.int64, np.complex128])
@pytest.mark.parametrize("shape,dims", [((1 << 20,), None), ((1 << 20) + 3, None), ((512, 1000), 1), ((512, 1000), 2), ((512, 1000), None),
                                        ((3, 100_000), 1), ((3, 100_000), 2), ((64, 3, 5, 7), (2, 3)), ((64, 3, 5, 7), (1, 4)),
                                        ((16, 1, 33), (1, 2)), ((7, 1, 1), 2)])
def test_element_sizes_and_unit_path(rk, orc, dtype, shape, dims):
    x = _rand(np.random.default_rng(5), dtype, shape)
    xd = rk.ROCArray(x)
    want = orc.reverse(x, dims=dims)
    _same(rk.Array(rk.reverse(xd, dims=dims)), want)
    _same(rk.Array(xd), x)                                   # the source is untouched
    _same(rk.Array(rk.reverse_(xd, dims=dims)), want)
    _same(rk.Array(rk.reverse_(xd, dims=dims)), x)           # an involution


def test_argument_errors_and_views(rk, orc):
    xd = rk.ROCArray(np.arange(10, dtype=np.int32))
    with pytest.raises(ValueError):
        rk.reverse(xd, dims=2)
    with pytest.raises(ValueError):
        rk.reverse_(xd, dims=0)
    with pytest.raises(IndexError):
        rk.reverse(xd, 0, 5)
    x = np.arange(1001, dtype=np.int32)
    d = rk.ROCArray(x)
    v = d.view_range(2, 1001)                                # 4-byte offset: element path
    _same(rk.Array(rk.reverse(v)), x[1:][::-1].copy())
    assert len(rk.reverse(rk.ROCArray(np.zeros(0, dtype=np.float32)))) == 0
    # reverse(x, start, stop) with an empty range is a copy
    _same(rk.Array(rk.reverse(xd, 5, 4)), np.arange(10, dtype=np.int32))
