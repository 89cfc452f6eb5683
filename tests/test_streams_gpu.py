"""Several streams at once, each with its own workspace: the boundary's contract is one workspace per stream, any
number of streams concurrently (Julia tasks each own a stream, src/tls.jl:71-86).  Calls are enqueued round-robin on
three streams without synchronising in between, so their kernels -- including the chained scans and the sort, whose
workgroups wait on one another through the workspace -- overlap on the device; every result is checked afterwards."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_three_streams_interleaved(rk, orc):
    rng = np.random.default_rng(51)
    streams = [torch.cuda.Stream() for _ in range(3)]
    n = (1 << 22) + 13
    jobs = []
    for k, s in enumerate(streams):
        with torch.cuda.stream(s):
            x = rng.integers(-1000, 1001, n, dtype=np.int32)
            f = rng.standard_normal(n).astype(np.float32)
            m = rng.random(n) < 0.3
            b = rng.integers(-10**6, 10**6, (300, 4099)).astype(np.int64)
            jobs.append(dict(x=x, f=f, m=m, b=b, dx=rk.ROCArray(x), df=rk.ROCArray(f), dm=rk.ROCArray(m), db=rk.ROCArray(b), out=[]))
    torch.cuda.synchronize()
    for it in range(3):                                   # enqueue without waiting: the streams run side by side
        for s, j in zip(streams, jobs):
            with torch.cuda.stream(s):
                j["out"].append((rk.cumsum(j["dx"]), rk.mapreduce("identity", "add", j["df"], dims=1), rk.cumsum(j["db"], dims=2),
                                 rk.sort(j["df"]), rk.findall(j["dm"]), rk.maximum(j["db"], dims=1)))
    torch.cuda.synchronize()
    for j in jobs:
        for cs, sm, c2, so, fa, mx in j["out"]:
            assert np.array_equal(rk.Array(cs), orc.cumsum(j["x"]))
            np.testing.assert_allclose(rk.Array(sm)[0], j["f"].astype(np.float64).sum(), rtol=1e-5, atol=1e-2)
            assert np.array_equal(rk.Array(c2), np.cumsum(j["b"], axis=1))
            assert np.array_equal(rk.Array(so), np.sort(j["f"]))
            assert np.array_equal(rk.Array(fa), np.nonzero(j["m"])[0] + 1)
            assert np.array_equal(rk.Array(mx), j["b"].max(axis=0, keepdims=True))


def test_two_streams_beyond_residency(rk, orc):
    """Two streams, each with grids far larger than what is resident at once (8192 tiles of the 1-D scan, 3072 of the
    scan across rows, 512 of the select), enqueued without waiting in between, with the default wait budget: tiles of
    two ordered grids share the compute units while each waits on predecessors of its own grid.  The 1-D scan and the
    select cannot stall (a tile that waits too long resolves its prefix alone); the chains of the scan across rows stay
    on one XCD each, where workgroups start in index order.  Integers, so every result is exact."""
    rng = np.random.default_rng(52)
    streams = [torch.cuda.Stream() for _ in range(2)]
    n = 1 << 26
    jobs = []
    for s in streams:
        with torch.cuda.stream(s):
            x = rng.integers(-1000, 1001, n, dtype=np.int32)
            b = rng.integers(-1000, 1001, (4096, 16384), dtype=np.int32)
            m = rng.random(n) < 0.25
            jobs.append(dict(x=x, b=b, m=m, dx=rk.ROCArray(x), db=rk.ROCArray(b), dm=rk.ROCArray(m), out=[]))
    torch.cuda.synchronize()
    for it in range(2):
        for s, j in zip(streams, jobs):
            with torch.cuda.stream(s):
                j["out"].append((rk.cumsum(j["dx"]), rk.cumsum(j["db"], dims=2), rk.findall(j["dm"])))
    torch.cuda.synchronize()
    for j in jobs:
        want_x = orc.cumsum(j["x"])
        want_b = np.cumsum(j["b"], axis=1, dtype=np.int32)
        want_m = np.nonzero(j["m"])[0] + 1
        for cs, c2, fa in j["out"]:
            assert np.array_equal(rk.Array(cs), want_x)
            assert np.array_equal(rk.Array(c2), want_b)
            assert np.array_equal(rk.Array(fa), want_m)
