"""GPU parity of findall / logical indexing masks (src/kernels/indexing.jl:8-36, test/hip_rocarray/indexing.jl:5-18)
against the oracle, through the C ABI: the one-pass stream compaction (rk_findall) and the reference's own
cumsum + scatter sequence (rk_accumulate + rk_findall_scatter).  Indices are bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _check(rk, orc, m):
    from amdgpu_jl_amd.indexing import findall_two_pass
    want = orc.findall(m)
    d = rk.ROCArray(m)
    for fn in (rk.findall, findall_two_pass):
        got = rk.Array(fn(d))
        assert got.dtype == np.int64
        assert np.array_equal(got if m.ndim == 1 else got.T, want), fn.__name__


@pytest.mark.parametrize("n", [1, 2, 15, 16, 17, 1000, 65535, 65536, 65537, 131072, 1_000_003, (1 << 22) + 5])
@pytest.mark.parametrize("density", [0.0, 0.03, 0.5, 1.0])
def test_findall_vector(rk, orc, n, density):
    _check(rk, orc, np.random.default_rng(n).random(n) < density)


@pytest.mark.parametrize("shape", [(16,), (1, 16), (3, 1, 16), (33, 65), (257, 300, 7), (2, 3, 4, 5, 6, 7), (70000, 3), (1, 1, 200_000)])
def test_findall_shapes(rk, orc, shape):
    # test/hip_rocarray/indexing.jl:5-18 shapes first
    _check(rk, orc, np.random.default_rng(7).random(shape) < 0.5)


def test_findall_unaligned_view_and_patterns(rk, orc):
    b = np.random.default_rng(3).random(200_001) < 0.4
    d = rk.ROCArray(b)
    v = d.view_range(2, 200_001)                               # byte offset 1: the scalar load path
    assert np.array_equal(rk.Array(rk.findall(v)), orc.findall(b[1:]))
    for pat in (np.arange(300_000) % 64 == 63, np.arange(300_000) % 1024 < 3, np.arange(300_000) >= 299_999):
        _check(rk, orc, pat)


def test_findall_repeated_calls_share_the_workspace_with_scans(rk, orc):
    rng = np.random.default_rng(11)
    for it in range(8):
        n = int(rng.integers(70_000, 900_000))
        b = rng.random(n) < rng.random()
        assert np.array_equal(rk.Array(rk.findall(rk.ROCArray(b))), orc.findall(b)), it
        x = rng.integers(-100, 100, n, dtype=np.int32)
        assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(x))), orc.cumsum(x)), it


def test_findall_full_size_and_count_out(rk, orc):
    import torch
    from amdgpu_jl_amd import _lib as L
    from amdgpu_jl_amd.array import workspace, stream_ptr
    n = 1 << 26
    b = np.random.default_rng(5).random(n) < 0.25
    d = rk.ROCArray(b)
    total = int(b.sum())
    ys = rk.ROCArray(dims=(total,), dtype=np.int64)
    cnt = rk.ROCArray(dims=(1,), dtype=np.int64)
    shape = L.shape_array((n,))
    ws, ws_bytes = workspace(L.lib.rk_workspace_bytes(L.RK_KIND_FINDALL, L.RK_U8, 1, shape, 0))
    L.check(L.lib.rk_findall(d.ptr, 1, shape, ys.ptr, cnt.ptr, ws, ws_bytes, stream_ptr()), "rk_findall")
    assert int(rk.Array(cnt)[0]) == total
    assert np.array_equal(rk.Array(ys), np.nonzero(b)[0] + 1)
    # selection x[m] == x[findall(m)] (test/hip_rocarray/indexing.jl:8)
    x = np.random.default_rng(6).integers(-2**31, 2**31 - 1, 1 << 20, dtype=np.int32)
    m = np.random.default_rng(7).random(1 << 20) < 0.5
    idx = rk.Array(rk.findall(rk.ROCArray(m)))
    assert np.array_equal(x[idx - 1], x[m])


@pytest.mark.parametrize("dtype", [np.int32, np.float64, np.int16, np.bool_, np.complex128])
def test_selection_by_mask(rk, orc, dtype):
    # test/hip_rocarray/indexing.jl:5-18: x[m], x[:, m], x[:, :, m]
    rng = np.random.default_rng(12)
    def rand(shape):
        return (rng.random(shape) * 1000).astype(dtype) if np.dtype(dtype).kind != "b" else rng.random(shape) < 0.5
    for n in (16, 100_003):
        m = rng.random(n) < 0.5
        md = rk.ROCArray(m)
        for shape in ((n,), (1, n), (3, 1, n), (7, n)):
            x = rand(shape)
            got = rk.Array(rk.getindex_mask(rk.ROCArray(x), md))
            assert np.array_equal(got, x[..., m])
    x = rand((33, 65))
    m2 = rng.random((33, 65)) < 0.3
    got = rk.Array(rk.getindex_mask(rk.ROCArray(x), rk.ROCArray(m2)))
    assert np.array_equal(got, x.reshape(-1, order="F")[m2.reshape(-1, order="F")])        # column-major order of the hits
    with pytest.raises(IndexError):
        rk.getindex_mask(rk.ROCArray(x), rk.ROCArray(np.ones(5, dtype=bool)))
    assert rk.getindex_mask(rk.ROCArray(x), rk.ROCArray(np.zeros((33, 65), dtype=bool))).dims == (0,)


def test_the_paths_the_tunables_select():
    """RK_SELECT_ORDERED=0 (persistent workgroups fed by a tile counter) and RK_SCAN_DYNAMIC_IDS=1 (the same for the
    long scans) are read once per process, so they are exercised in a child process: findall and a long cumsum against
    numpy, several calls on one workspace."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = r'''
import sys
sys.path.insert(0, %r)
import numpy as np
from __graft_entry__ import load_package
rk = load_package()
rng = np.random.default_rng(5)
for n, dens in ((1 << 21) + 77, 0.3), ((1 << 22), 0.01), (300_000, 1.0), (5, 0.5):
    m = rng.random(n) < dens
    got = rk.Array(rk.findall(rk.ROCArray(m)))
    assert np.array_equal(got, np.flatnonzero(m) + 1), (n, dens)
m = rng.random((257, 3001)) < 0.4
got = rk.Array(rk.findall(rk.ROCArray(m)))
want = np.argwhere(m.T)[:, ::-1] + 1                  # column-major order of the hits
assert np.array_equal(got.T, want)
x = rng.integers(-100, 100, size=(1 << 22) + 3).astype(np.int32)
for _ in range(3):
    assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(x))), np.cumsum(x, dtype=np.int32))
print("child ok")
''' % root
    env = dict(os.environ, RK_SELECT_ORDERED="0", RK_SCAN_DYNAMIC_IDS="1")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert out.returncode == 0 and "child ok" in out.stdout, out.stdout[-2000:] + out.stderr[-2000:]
