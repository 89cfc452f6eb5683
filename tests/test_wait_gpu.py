"""Bounded waits: a look-back that cannot complete helps itself (single-pass scan of long lines, one-pass findall:
exact results whatever happens) or gives up and records it (the other kernels); every kernel exits.

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


def _alone_count(ws):
    """WsHeader::alone: tiles that stopped waiting and resolved their look-back by themselves."""
    return int(ws[12:16].cpu().numpy().view(np.uint32)[0])


@pytest.mark.parametrize("n", [(1 << 24) + 4096, 1 << 26])
def test_ordered_scan_helps_itself(rk, orc, tiny_budget, n):
    """The single-pass scan of long lines never gives up: a tile whose patience (here: one poll) runs out computes what
    its predecessors have not published from the input.  The result is exact and the status clean."""
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(15)
    h = rng.integers(-1000, 1001, n, dtype=np.int32)
    x = rk.ROCArray(h)
    out = rk.ROCArray(dims=x.dims, dtype=np.int32)
    ws = _fresh_workspace(L, 16 << 20)
    want = orc.accumulate("add", h, dims=1)
    for _ in range(3):
        out.buf.zero_()
        assert _scan(L, rk, x, out, ws) == 0
        assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
        assert np.array_equal(rk.Array(out), want)
    assert _alone_count(ws) > 0                                  # the path under test was taken
    # Float32 and max: the same path with another operator and rounding (tolerance of the scans)
    f = rng.random(n, dtype=np.float32)
    xf = rk.ROCArray(f)
    of = rk.ROCArray(dims=xf.dims, dtype=np.float32)
    assert L.lib.rk_accumulate(L.RK_OP_ADD, xf.code, of.code, xf.ptr, of.ptr, 1, L.shape_array(xf.dims), 1, 1, None,
                               ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    np.testing.assert_allclose(rk.Array(of), np.cumsum(f, dtype=np.float64), rtol=1e-4)
    assert L.lib.rk_accumulate(L.RK_OP_MAX, x.code, out.code, x.ptr, out.ptr, 1, L.shape_array(x.dims), 1, 1, None,
                               ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert np.array_equal(rk.Array(out), np.maximum.accumulate(h))
    assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
def test_packed_ordered_scan_helps_itself(rk, orc, tiny_budget, dtype):
    """The same for the packed tiles of 1- and 2-byte integers (a tile is 128 KiB of elements; the aggregates a tile
    computes for its predecessors are read from the input in the widened way)."""
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(17)
    n = (1 << 24) + 4096
    h = rng.integers(-100, 101, n).astype(dtype)
    x = rk.ROCArray(h)
    out = rk.ROCArray(dims=x.dims, dtype=dtype)
    ws = _fresh_workspace(L, 16 << 20)
    for op, code in (("add", L.RK_OP_ADD), ("max", L.RK_OP_MAX)):
        out.buf.zero_()
        assert L.lib.rk_accumulate(code, x.code, out.code, x.ptr, out.ptr, 1, L.shape_array(x.dims), 1, 1, None,
                                   ws.data_ptr(), ws.numel(), stream_ptr()) == 0
        assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
        assert np.array_equal(rk.Array(out), orc.accumulate(op, h, dims=1).astype(dtype))
    assert _alone_count(ws) > 0


@pytest.mark.parametrize("dtype", [np.int64, np.float64, np.bool_])
def test_ordered_scan_of_8_byte_values_helps_itself(rk, orc, tiny_budget, dtype):
    """8-byte values (and Bool -> Int64) run the same single-pass kernel: with a patience of one poll the tiles resolve
    their prefixes alone, the result is exact and the status clean."""
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(18)
    n = (1 << 23) + 2048
    h = (rng.random(n) < 0.5) if dtype == np.bool_ else rng.integers(-1000, 1001, n).astype(dtype)
    out_dtype = np.int64 if dtype == np.bool_ else dtype
    x = rk.ROCArray(h)
    out = rk.ROCArray(dims=x.dims, dtype=out_dtype)
    ws = _fresh_workspace(L, 16 << 20)
    assert L.lib.rk_accumulate(L.RK_OP_ADD, x.code, out.code, x.ptr, out.ptr, 1, L.shape_array(x.dims), 1, 1, None,
                               ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert np.array_equal(rk.Array(out), np.cumsum(h, dtype=out_dtype))        # integer-valued: exact in Float64 too
    assert _alone_count(ws) > 0


def test_ordered_scan_at_odd_addresses_helps_itself(rk, orc, tiny_budget):
    """Lines that start at odd addresses: the tiles that help themselves read their predecessors' elements with vectors
    at element-aligned addresses."""
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(19)
    h = rng.integers(-1000, 1001, ((1 << 21) + 1, 9), dtype=np.int32)     # nine lines of 65 tiles, every line at another alignment
    x = rk.ROCArray(h)
    out = rk.ROCArray(dims=x.dims, dtype=np.int32)
    ws = _fresh_workspace(L, 16 << 20)
    assert _scan(L, rk, x, out, ws, dims=1) == 0
    assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert np.array_equal(rk.Array(out), orc.accumulate("add", h, dims=1))
    assert _alone_count(ws) > 0


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.int16])
def test_ordered_scan_in_place_helps_itself(rk, orc, tiny_budget, dtype):
    """In place (out is in) a tile that helps itself reads elements that their own tile may be about to overwrite with its
    results: it takes what it computed only if that tile has still not published anything when the reads are done, and
    the tile's own aggregate otherwise.  Several rounds, a patience of one poll, exact results every time."""
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(20)
    n = (1 << 24) + 4096
    h = rng.integers(-100, 101, n).astype(dtype)
    want = orc.accumulate("add", h, dims=1).astype(dtype)
    ws = _fresh_workspace(L, 16 << 20)
    alone = 0
    for _ in range(6):
        y = rk.ROCArray(h)
        assert L.lib.rk_accumulate(L.RK_OP_ADD, y.code, y.code, y.ptr, y.ptr, 1, L.shape_array(y.dims), 1, 1, None,
                                   ws.data_ptr(), ws.numel(), stream_ptr()) == 0
        assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
        assert np.array_equal(rk.Array(y), want)
        alone = _alone_count(ws)
    assert alone > 0


def test_ordered_scan_of_many_lines_helps_itself(rk, orc, tiny_budget):
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(16)
    h = rng.integers(-1000, 1001, (1 << 21, 9), dtype=np.int32)     # nine lines of 64 tiles of 128 KiB each
    x = rk.ROCArray(h)
    out = rk.ROCArray(dims=x.dims, dtype=np.int32)
    ws = _fresh_workspace(L, 16 << 20)
    assert _scan(L, rk, x, out, ws, dims=1) == 0
    assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
    assert np.array_equal(rk.Array(out), orc.accumulate("add", h, dims=1))
    assert _alone_count(ws) > 0


def test_ordered_findall_helps_itself(rk, orc, tiny_budget):
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(17)
    for n in ((1 << 24) + 77, 1 << 27):
        b = rng.random(n) < 0.05
        db = rk.ROCArray(b)
        want = np.flatnonzero(b) + 1
        ys = rk.ROCArray(dims=(want.size,), dtype=np.int64)
        shp = L.shape_array(b.shape)
        ws = _fresh_workspace(L, int(L.lib.rk_workspace_bytes(L.RK_KIND_FINDALL, L.RK_U8, 1, shp, 0)))
        for _ in range(2):
            ys.buf.zero_()
            assert L.lib.rk_findall(db.ptr, 1, shp, ys.ptr, None, ws.data_ptr(), ws.numel(), stream_ptr()) == 0
            assert L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == 0
            assert np.array_equal(rk.Array(ys), want)
        assert _alone_count(ws) > 0


def test_give_up_is_scoped_to_its_call(rk, orc, tiny_budget):
    """A give-up marks the workspace with the epoch of ITS call: a later call on the same workspace (not prepared again)
    neither follows the old mark nor clears it."""
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(8)
    h = rng.integers(-1000, 1001, (2048, 8192), dtype=np.int32)  # scanned across rows: a kernel that cannot help itself
    x = rk.ROCArray(h)
    out = rk.ROCArray(dims=x.dims, dtype=np.int32)
    ws = _fresh_workspace(L, 16 << 20)
    want = orc.accumulate("add", h, dims=2)
    gave_up = False
    for _ in range(4):                                           # a budget of one poll: some tile nearly always exceeds it
        assert _scan(L, rk, x, out, ws, dims=2) == 0
        if L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr()) == L.RK_ERR_WAIT:
            gave_up = True
            break
    L.lib.rk_set_wait_budget(0)
    # NOT prepared again: with the default budget the next call must be right although the old mark is still there
    out.buf.zero_()
    assert _scan(L, rk, x, out, ws, dims=2) == 0
    st = L.lib.rk_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr())
    assert st == (L.RK_ERR_WAIT if gave_up else 0)               # the mark stays until the workspace is prepared again
    assert np.array_equal(rk.Array(out), want)


def test_mirror_raises_on_give_up(rk, orc, tiny_budget):
    """Through the host mirror: `Array(cumsum(x))` is either right or raises WaitError -- never a wrong array with a
    clean status -- and after the exception the same call works."""
    L = tiny_budget
    rng = np.random.default_rng(9)
    h = rng.integers(-1000, 1001, (2048, 8192), dtype=np.int32)
    x = rk.ROCArray(h)
    want = np.cumsum(h, axis=1, dtype=np.int32)
    raised = 0
    for _ in range(4):
        y = rk.cumsum(x, dims=2)
        try:
            got = rk.Array(y)
        except L.WaitError as e:
            assert e.status == L.RK_ERR_WAIT
            raised += 1
            continue
        assert np.array_equal(got, want)
    L.lib.rk_set_wait_budget(0)
    assert np.array_equal(rk.Array(rk.cumsum(x, dims=2)), want)  # the mirror prepared the workspace again
    # findall and a small sort go the same way
    L.lib.rk_set_wait_budget(1)
    b = rng.random(1 << 24) < 0.3
    db = rk.ROCArray(b)
    k = rng.standard_normal(1 << 20).astype(np.float32)
    for _ in range(2):
        try:
            assert np.array_equal(rk.Array(rk.findall(db)), np.flatnonzero(b) + 1)
        except L.WaitError:
            pass
        try:
            assert np.array_equal(rk.Array(rk.sort(rk.ROCArray(k))), np.sort(k))
        except L.WaitError:
            pass
    L.lib.rk_set_wait_budget(0)
    assert np.array_equal(rk.Array(rk.findall(db)), np.flatnonzero(b) + 1)
    assert np.array_equal(rk.Array(rk.sort(rk.ROCArray(k))), np.sort(k))


def test_static_scratch_reports_and_recovers(rk, orc, tiny_budget):
    L = tiny_budget
    from amdgpu_jl_amd.array import stream_ptr
    rng = np.random.default_rng(10)
    h = rng.integers(-1000, 1001, 1 << 24, dtype=np.int32)
    x = rk.ROCArray(h)
    out = rk.ROCArray(dims=x.dims, dtype=np.int32)
    want = orc.cumsum(h)

    def call():
        return L.lib.rk_accumulate_static(L.RK_OP_ADD, x.code, out.code, x.ptr, out.ptr, 1, L.shape_array(x.dims), 1, 1, None, stream_ptr())
    L.lib.rk_set_wait_budget(0)
    assert call() == 0                                           # the first call on the device prepares the array
    assert L.lib.rk_accumulate_static_status(stream_ptr()) == 0
    L.lib.rk_set_wait_budget(1)
    assert call() == 0
    st = L.lib.rk_accumulate_static_status(stream_ptr())
    assert st in (0, L.RK_ERR_WAIT)
    if st == 0:
        assert np.array_equal(rk.Array(out), want)
    L.lib.rk_set_wait_budget(0)
    assert L.lib.rk_accumulate_static_status(stream_ptr()) == 0  # reported once, prepared again by the status call
    assert call() == 0
    assert L.lib.rk_accumulate_static_status(stream_ptr()) == 0
    assert np.array_equal(rk.Array(out), want)


def test_status_argument_checks(rk):
    import ctypes as C
    from amdgpu_jl_amd import _lib as L
    assert L.lib.rk_workspace_status(None, 1 << 24, None) == L.RK_ERR_INVALID_ARGUMENT
    assert L.lib.rk_workspace_status(C.c_void_p(0x1001), 1 << 24, None) == L.RK_ERR_WORKSPACE
    assert L.lib.rk_sort_status(None, 1 << 20, None) == L.RK_ERR_INVALID_ARGUMENT
    prev = L.lib.rk_set_wait_budget(12345)
    assert L.lib.rk_set_wait_budget(prev) == 12345
