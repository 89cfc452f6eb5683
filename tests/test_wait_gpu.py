"""Bounded waits: a look-back that cannot complete gives up, records it, and every kernel still exits.

The condition is forced from the host: rk_set_wait_budget(1) lets a wait spend ONE unsuccessful poll, which in a scan of
thousands of tiles some tile always exceeds (a predecessor's aggregate is not there yet at the first look).  The
kernels run to their end with meaningless results, rk_workspace_status / rk_sort_status report RK_ERR_WAIT, and after
preparing the workspace again the same call is correct.  No kernel faults, traps or hangs here."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture()
def tiny_budget():
    from amdgpu_jl_amd import _lib as L
    prev = L.lib.rk_set_wait_budget(1)
    yield L
    L.lib.rk_set_wait_budget(prev)


def _fresh_workspace(L, nbytes):
    import torch
    from amdgpu_jl_amd.array import stream_ptr
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    assert ws.data_ptr() % 256 == 0
    assert L.lib.rk_workspace_init(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    return ws


def _scan(L, rk, x, out, ws, dims=1):
    from amdgpu_jl_amd.array import stream_ptr
    return L.lib.rk_accumulate(L.RK_OP_ADD, x.code, out.code, x.ptr, out.ptr, x.ndim, L.shape_array(x.dims), dims, 1, None,
                               ws.data_ptr(), ws.numel(), stream_ptr())


@pytest.mark.parametrize("shape,dims", [((1 << 24,), 1), ((2048, 8192), 2), ((64, 200_000), 2)])
def test_scan_gives_up_and_recovers(rk, orc, tiny_budget, shape, dims):
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(5)
    h = rng.integers(-1000, 1001, shape, dtype=np.int32)
    x = rk.ROCArray(h)
    out = rk.ROCArray(dims=x.dims, dtype=np.int32)
    ws = _fresh_workspace(L, 16 << 20)
    assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert _scan(L, rk, x, out, ws, dims) == 0                   # launches fine; the kernels exit on their own
    st = L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr())      # synchronises
    want = orc.accumulate("add", h, dims=dims)
    if st == 0:
        assert np.array_equal(rk.Array(out), want)               # nobody had to wait twice: then the result must be right
    else:
        assert st == L.RK_ERR_WAIT
        assert L.lib.rk_status_string(st).startswith(b"RK_ERR_WAIT")
    # the default budget again, the workspace prepared again: correct, and the status is clean
    L.lib.rk_set_wait_budget(0)
    assert L.lib.rk_workspace_init(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert _scan(L, rk, x, out, ws, dims) == 0
    assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert np.array_equal(rk.Array(out), want)


def test_findall_gives_up_and_recovers(rk, orc, tiny_budget):
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(6)
    # one-pass findall: chained look-back over tiles of 256 Ki Bools.  A prefix cut short by a give-up is a partial
    # sum of true counts, i.e. too small, so every index still lands inside `ys`.
    b = rng.random(1 << 24) < 0.3
    db = rk.ROCArray(b)
    cnt = int(np.count_nonzero(b))
    ys = rk.ROCArray(dims=(cnt,), dtype=np.int64)
    shp = L.shape_array(b.shape)
    ws = _fresh_workspace(L, int(L.lib.rk_workspace_bytes(L.RK_KIND_FINDALL, L.RK_U8, 1, shp, 0)))
    assert L.lib.rk_findall(db.ptr, 1, shp, ys.ptr, None, ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    st = L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr())
    assert st in (0, L.RK_ERR_WAIT)
    if st == 0:
        assert np.array_equal(rk.Array(ys), np.flatnonzero(b) + 1)
    L.lib.rk_set_wait_budget(0)
    assert L.lib.rk_workspace_init(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert L.lib.rk_findall(db.ptr, 1, shp, ys.ptr, None, ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert np.array_equal(rk.Array(ys), np.flatnonzero(b) + 1)


def test_sort_gives_up_and_recovers(rk, orc, tiny_budget):
    import torch
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(7)
    # 2^20 keys: 256 tiles chained by look-back.  After a give-up no further tile starts and every store is kept inside
    # the arrays (a pass that follows one with holes reads keys the histograms never counted).
    k = rng.standard_normal(1 << 20).astype(np.float32)
    dk = rk.ROCArray(k)
    tmp = torch.empty(int(L.lib.rk_sort_tmp_bytes(L.RK_F32, k.size, 0)), dtype=torch.uint8, device="cuda")
    assert L.lib.rk_sort(L.RK_F32, dk.ptr, k.size, 0, tmp.data_ptr(), tmp.numel(), stream_ptr()) == 0
    st = L.lib.rk_sort_status(tmp.data_ptr(), tmp.numel(), stream_ptr())
    assert st in (0, L.RK_ERR_WAIT)
    if st == 0:
        assert np.array_equal(rk.Array(dk), np.sort(k))
    L.lib.rk_set_wait_budget(0)
    dk = rk.ROCArray(k)
    assert L.lib.rk_sort(L.RK_F32, dk.ptr, k.size, 0, tmp.data_ptr(), tmp.numel(), stream_ptr()) == 0
    assert L.lib.rk_sort_status(tmp.data_ptr(), tmp.numel(), stream_ptr()) == 0
    assert np.array_equal(rk.Array(dk), np.sort(k))


def test_status_argument_checks(rk):
    import ctypes as C
    from amdgpu_jl_amd import _lib as L
    assert L.lib.rk_workspace_status(None, 1 << 24, None) == L.RK_ERR_INVALID_ARGUMENT
    assert L.lib.rk_workspace_status(C.c_void_p(0x1001), 1 << 24, None) == L.RK_ERR_WORKSPACE
    assert L.lib.rk_sort_status(None, 1 << 20, None) == L.RK_ERR_INVALID_ARGUMENT
    prev = L.lib.rk_set_wait_budget(12345)
    assert L.lib.rk_set_wait_budget(prev) == 12345
