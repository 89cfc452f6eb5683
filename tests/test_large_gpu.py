"""More than 2^31 elements: the 64-bit index paths of the streaming kernels.  Inputs are generated and results
are checked on the device (closed forms, in chunks), because arrays of this size do not fit a host copy."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

N = (1 << 31) + (1 << 20) + 3
CHUNK = 1 << 26


def _wrap(rk, t, dtype):
    import torch
    return rk.ROCArray(buf=t.view(torch.uint8).reshape(-1), dims=(t.numel(),), dtype=dtype)


def test_sum_and_findmax_beyond_2_31(rk):
    import torch
    x = torch.ones(N, dtype=torch.float32, device="cuda")
    d = _wrap(rk, x, np.float32)
    assert float(rk.sum(d)) == float(np.float32(N))         # the exact count rounded once to Float32 (rtol 1e-5 would allow more)
    x[N - 5] = 7.0
    v, i = rk.findmax(d)
    assert float(v) == 7.0 and int(i) == N - 4              # 1-based, beyond Int32
    del x, d
    torch.cuda.empty_cache()


def test_cumsum_beyond_2_31_wraps_like_int32(rk):
    import torch
    x = torch.ones(N, dtype=torch.int32, device="cuda")
    out = rk.cumsum(_wrap(rk, x, np.int32))
    got = out.buf.view(torch.int32)
    for lo in range(0, N, CHUNK):
        hi = min(lo + CHUNK, N)
        want = torch.arange(lo + 1, hi + 1, dtype=torch.int64, device="cuda").to(torch.int32)    # wraps mod 2^32
        assert bool((got[lo:hi] == want).all()), lo
    del x, out, got
    torch.cuda.empty_cache()


def test_broadcast_reverse_findall_beyond_2_31(rk):
    import torch
    x = torch.empty(N, dtype=torch.float32, device="cuda")
    for lo in range(0, N, CHUNK):
        hi = min(lo + CHUNK, N)
        x[lo:hi] = torch.arange(lo, hi, dtype=torch.int64, device="cuda").remainder(1 << 20).to(torch.float32)
    d = _wrap(rk, x, np.float32)
    z = rk.materialize(np.float32(2.0) * rk.lazy(d) + rk.lazy(d))
    r = rk.reverse(d)
    gz, gr = z.buf.view(torch.float32), r.buf.view(torch.float32)
    for lo in range(0, N, CHUNK):
        hi = min(lo + CHUNK, N)
        assert bool((gz[lo:hi] == 3.0 * x[lo:hi]).all()), lo
        assert bool((gr[lo:hi] == x[N - hi:N - lo].flip(0)).all()), lo
    del z, r, gz, gr
    m = (x == 5.0)                                           # one hit per 2^20 elements: 2049 hits
    del x, d
    torch.cuda.empty_cache()
    idx = rk.Array(rk.findall(_wrap(rk, m, np.bool_)))
    assert np.array_equal(idx, np.arange(5, N, 1 << 20, dtype=np.int64) + 1)


# Outer extents beyond 65535 (the limit of a grid's y and z axes) with lanes along the first dim: the shapes an
# earlier version refused with RK_ERR_TOO_LARGE.  Small arrays, checked against the oracle.
LONG_OUTER = [(64, 2, 70000), (64, 5, 70000), (100, 3, 111848), (256, 2, 65536)]


@pytest.mark.parametrize("shape", LONG_OUTER)
@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32])
def test_reduce_dims2_long_outer(rk, orc, shape, dtype):
    rng = np.random.default_rng(sum(shape))
    h = (rng.standard_normal(shape) * 100).astype(dtype)
    d = rk.ROCArray(h)
    got = rk.Array(rk.sum(d, dims=2))
    want = orc.mapreduce("identity", "add", h, dims=2)
    if np.dtype(dtype).kind == "f":
        np.testing.assert_allclose(got, want, rtol=1e-5 if dtype == np.float32 else 1e-12, atol=1e-3 if dtype == np.float32 else 1e-9)
    else:
        assert np.array_equal(got, want)
    v, i = rk.findmax(d, dims=2)
    ov, oi = orc.findmax(h, dims=2)
    assert np.array_equal(rk.Array(v), ov)
    assert np.array_equal(np.moveaxis(rk.Array(i), 0, -1), oi)


@pytest.mark.parametrize("shape", [(64, 64, 70000), (1000, 3, 112625), (2048, 4, 100000), (64, 300, 66000)])
def test_accumulate_dims2_long_outer(rk, orc, shape):
    rng = np.random.default_rng(sum(shape))
    h = rng.integers(-1000, 1001, shape, dtype=np.int32)
    got = rk.Array(rk.cumsum(rk.ROCArray(h), dims=2))
    assert np.array_equal(got, orc.accumulate("add", h, dims=2))
