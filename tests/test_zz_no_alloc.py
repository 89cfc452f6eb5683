"""rk_accumulate_static (bookkeeping in the library's own device array, no workspace argument, no allocation)
against rk_accumulate on the same inputs AND against the CPU oracle, through the C ABI.

Bar: integer scans bit-exact (both ways); Float32 within rtol 1e-4 of the oracle's Float64 scan and of each other (both
are Float32 scans whose look-back association order depends on timing, so they need not agree to the bit).  The calls
run with torch's allocator watched: the entry point must not change the device memory the process holds.  Every case makes two calls in a row on the
one shared array, the second on a smaller input, so that state left by the first call would show."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(rk, x, op="add", dims=1, inclusive=True, init=None, out_dtype=None):
    from amdgpu_jl_amd import _lib as L
    from amdgpu_jl_amd.array import stream_ptr
    from amdgpu_jl_amd.mapreduce import _OP, _scalar_buffer
    A = rk.ROCArray(x)
    out_dtype = np.dtype(out_dtype or x.dtype)
    want = rk.ROCArray(dims=A.dims, dtype=out_dtype)
    rk.accumulate_(op, want, A, dims=dims, init=init, inclusive=inclusive)          # rk_accumulate with a caller workspace
    got = rk.ROCArray(dims=A.dims, dtype=out_dtype)
    got.buf.fill_(0xA5)
    ibuf = _scalar_buffer(init, out_dtype)
    shape = L.shape_array(A.dims)
    import torch
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    st = L.lib.rk_accumulate_static(_OP[op], A.code, got.code, A.ptr, got.ptr, A.ndim, shape, dims,
                                    1 if inclusive else 0, ibuf, stream_ptr())
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert st == 0, L.lib.rk_status_string(st)
    assert free1 == free0, "rk_accumulate_static changed the free device memory: it must not allocate"
    return rk.Array(got), rk.Array(want)


def _oracle(orc, x, op="add", dims=1, inclusive=True, init=None, out_dtype=None):
    xx = x.astype(out_dtype) if out_dtype is not None else x
    return orc.accumulate(op, xx, dims=dims, init=init, inclusive=inclusive)


def _check(got, want):
    if want.dtype.kind == "f":
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-3)
    else:
        assert np.array_equal(got, want)


# (first shape, second smaller shape, dims): long lines (chained look-back: counter + descriptors), scan across rows
# with slices (slice totals in the scratch area), narrow inner (tile totals), one-tile lines (no bookkeeping)
CASES = [
    ((1 << 22) + 77, 300_001, 1),
    ((4096, 2048), (1024, 100), 2),
    ((3, 400_000), (3, 9_000), 2),
    ((70_000, 40), (40_000, 3), 1),
    ((5000,), (17,), 1),
]


@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.int64])
@pytest.mark.parametrize("first,second,dims", CASES)
def test_static_matches_workspace(rk, orc, first, second, dims, dtype):
    rng = np.random.default_rng(11)
    for shape in (first, second):
        shape = (shape,) if isinstance(shape, int) else shape
        if np.dtype(dtype).kind == "f":
            x = rng.random(shape, dtype=np.float32).astype(dtype)
        else:
            x = rng.integers(-1000, 1001, shape).astype(dtype)
        got, want = _both(rk, x, dims=dims)
        _check(got, want)
        _check(got, _oracle(orc, x, dims=dims).astype(got.dtype))


def test_static_exclusive_init_and_bool_counts(rk, orc):
    rng = np.random.default_rng(12)
    x = rng.integers(-5, 6, 1_000_003).astype(np.int32)
    for n in (x.size, 70_001):
        got, want = _both(rk, x[:n].copy(), op="max", inclusive=False, init=-3)
        _check(got, want)
        _check(got, _oracle(orc, x[:n], op="max", inclusive=False, init=-3))
    b = rng.random(3_000_000) < 0.3
    for n in (b.size, 100_000):
        got, want = _both(rk, b[:n].copy(), out_dtype=np.int64)
        _check(got, want)
        assert np.array_equal(got, np.cumsum(b[:n], dtype=np.int64))
        assert got[-1] == np.count_nonzero(b[:n])


def test_static_rejects_what_does_not_fit_and_empty(rk):
    from amdgpu_jl_amd import _lib as L
    from amdgpu_jl_amd.array import stream_ptr
    # 2^26 lines of 16385 Float64: one descriptor set per line exceeds the 16 MiB array; rejected before any device work
    shape = L.shape_array((16385, 1 << 26))
    st = L.lib.rk_accumulate_static(L.RK_OP_ADD, L.RK_F64, L.RK_F64, C.c_void_p(256), C.c_void_p(512), 2, shape, 1, 1, None, stream_ptr())
    assert st == L.RK_ERR_TOO_LARGE
    assert L.lib.rk_workspace_bytes(L.RK_KIND_ACCUMULATE, L.RK_F64, 2, shape, 1) > L.RK_STATIC_SCRATCH_BYTES
    st = L.lib.rk_accumulate_static(L.RK_OP_ADD, L.RK_F32, L.RK_F32, None, None, 1, L.shape_array((0,)), 1, 1, None, stream_ptr())
    assert st == 0
