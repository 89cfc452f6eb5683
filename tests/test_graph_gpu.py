"""Replays of a captured HIP graph: every kernel of the library keeps its cross-workgroup state (tickets,
scan epoch, descriptors) on the device, so a captured launch sequence must give the oracle's result on
every replay, with new input contents each time and eager work between the replays."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _upload(dst, host):
    flat = np.ascontiguousarray(host.reshape(-1, order="F")).view(np.uint8)
    dst.buf[: flat.size].copy_(torch.from_numpy(flat.copy()).to(dst.buf.device))


def test_graph_replays_match_oracle(rk, orc):
    from amdgpu_jl_amd.accumulate import plan_accumulate
    from amdgpu_jl_amd.broadcast import plan_materialize, lazy, exp
    from amdgpu_jl_amd.mapreduce import plan_findmax, plan_mapreducedim

    n = (1 << 21) + 77                      # several look-back tiles, ragged tail
    shape2 = (192, 4100)                    # scan across rows: totals, scan of the totals, carried slices
    rng = np.random.default_rng(41)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        # arrays, workspaces and prepared calls are made before the capture: a workspace allocated during a capture
        # would not belong to the graph (rk_workspace_init itself is a fill kernel and could be captured)
        xf = rk.ROCArray(dims=(n,), dtype=np.float32)
        xi = rk.ROCArray(dims=(n,), dtype=np.int32)
        m2 = rk.ROCArray(dims=shape2, dtype=np.int32)
        r_sum = rk.ROCArray(dims=(1,), dtype=np.float32)
        r_scan = rk.ROCArray(dims=(n,), dtype=np.int32)
        r_scan2 = rk.ROCArray(dims=shape2, dtype=np.int32)
        r_bc = rk.ROCArray(dims=(n,), dtype=np.float32)
        r_val = rk.ROCArray(dims=(1, shape2[1]), dtype=np.int32)
        r_idx = rk.ROCArray(dims=(2, 1, shape2[1]), dtype=np.int64)
        r_row = rk.ROCArray(dims=(shape2[0], 1), dtype=np.int64)
        calls = [
            plan_mapreducedim("identity", "add", r_sum, xf),
            plan_accumulate("add", r_scan, xi),
            plan_accumulate("add", r_scan2, m2, dims=2),
            plan_materialize(r_bc, np.float32(0.5) * lazy(xf) + lazy(xf) * exp(lazy(xf))),
            plan_findmax(m2, r_val, r_idx, 1),
            plan_mapreducedim("identity", "add", r_row, m2),
        ]
        for c in calls:                     # one eager pass: first-use set-up happens outside the capture
            c()
    side.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for c in calls:
            c()

    for replay in range(4):
        hf = rng.standard_normal(n).astype(np.float32)
        hi = rng.integers(-1000, 1001, n, dtype=np.int32)
        h2 = rng.integers(-10**6, 10**6, shape2, dtype=np.int32)
        _upload(xf, hf)
        _upload(xi, hi)
        _upload(m2, h2)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_allclose(rk.Array(r_sum)[0], hf.astype(np.float64).sum(), rtol=1e-5, atol=1e-2, err_msg=f"replay {replay}")
        assert np.array_equal(rk.Array(r_scan), orc.cumsum(hi)), replay
        assert np.array_equal(rk.Array(r_scan2), orc.cumsum(h2, dims=2)), replay
        h64 = hf.astype(np.float64)
        ref = 0.5 * h64 + h64 * np.exp(h64)
        np.testing.assert_allclose(rk.Array(r_bc), ref, rtol=1e-5, atol=1e-5, err_msg=f"replay {replay}")
        assert np.array_equal(rk.Array(r_val)[0], h2.max(axis=0)), replay
        assert np.array_equal(rk.Array(r_idx)[0, 0], h2.argmax(axis=0) + 1), replay
        assert np.array_equal(rk.Array(r_row)[:, 0], h2.astype(np.int64).sum(axis=1)), replay
        # eager work through the default stream's workspace between the replays
        assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(hi[:300_000]))), np.cumsum(hi[:300_000], dtype=np.int32))


def test_graph_replays_of_findall_reverse_permutedims_sort(rk, orc):
    import ctypes as C
    from amdgpu_jl_amd import _lib as L
    from amdgpu_jl_amd.array import workspace, stream_ptr

    n, shape2 = 300_007, (130, 257)
    rng = np.random.default_rng(43)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        mask = rk.ROCArray(dims=(n,), dtype=np.bool_)
        ys = rk.ROCArray(dims=(n,), dtype=np.int64)                # room for every element
        cnt = rk.ROCArray(dims=(1,), dtype=np.int64)
        keys = rk.ROCArray(dims=(n,), dtype=np.float32)
        perm = rk.ROCArray(dims=(n,), dtype=np.int64)
        m2 = rk.ROCArray(dims=shape2, dtype=np.int32)
        rev = rk.ROCArray(dims=shape2, dtype=np.int32)
        tr = rk.ROCArray(dims=shape2[::-1], dtype=np.int32)
        shp1, shp2 = L.shape_array((n,)), L.shape_array(shape2)
        p21 = (C.c_int32 * 2)(2, 1)
        ws, wsb = workspace(L.lib.rk_workspace_bytes(L.RK_KIND_FINDALL, L.RK_U8, 1, shp1, 0))
        tmp = torch.empty(int(L.lib.rk_sort_tmp_bytes(L.RK_F32, n, 1)), dtype=torch.uint8, device="cuda")

        def calls():
            s = stream_ptr()
            L.check(L.lib.rk_findall(mask.ptr, 1, shp1, ys.ptr, cnt.ptr, ws, wsb, s), "rk_findall")
            L.check(L.lib.rk_sortperm(L.RK_F32, keys.ptr, perm.ptr, n, 0, tmp.data_ptr(), tmp.numel(), s), "rk_sortperm")
            L.check(L.lib.rk_sort(L.RK_F32, keys.ptr, n, 1, tmp.data_ptr(), tmp.numel(), s), "rk_sort")
            L.check(L.lib.rk_reverse(m2.ptr, rev.ptr, 4, 2, shp2, 1, s), "rk_reverse")
            L.check(L.lib.rk_permutedims(m2.ptr, tr.ptr, 4, 2, shp2, p21, s), "rk_permutedims")
        mask.buf.zero_(); keys.buf.zero_(); m2.buf.zero_()
        calls()
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        calls()
    for replay in range(3):
        hm = rng.random(n) < 0.3
        hk = rng.standard_normal(n).astype(np.float32)
        h2 = rng.integers(-10**6, 10**6, shape2, dtype=np.int32)
        _upload(mask, hm); _upload(keys, hk); _upload(m2, h2)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        c = int(rk.Array(cnt)[0])
        assert c == int(hm.sum()), replay
        assert np.array_equal(rk.Array(ys)[:c], np.nonzero(hm)[0] + 1), replay
        assert np.array_equal(rk.Array(perm), orc.sortperm(hk)), replay
        assert np.array_equal(rk.Array(keys), orc.sort(hk, rev=True)), replay
        assert np.array_equal(rk.Array(rev), h2[::-1, :]), replay
        assert np.array_equal(rk.Array(tr), h2.T), replay
