"""The HIP path on the committed fixtures: the inputs tests/golden/make_golden.py draws (same seed, same order) go
through librk.so and must reproduce tests/golden/oracle_golden.json.

Tolerances: integers and indices bit-exact; Float32 sums rtol 1e-5, scans rtol 1e-4, broadcast with exp the mixed bound
1e-6 (|a x| + |y e^w|) + 1e-5 |ref|, `A .+ r .* c` within rtol 1e-6 of the Float64 values the fixture holds and
bit-exact against the un-fused Float32 evaluation of the same inputs on the host, volumerhs rtol 1e-4 plus 2e-6 of the
largest entry."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def golden():
    with open(os.path.join(HERE, "golden", "oracle_golden.json")) as fh:
        return json.load(fh)


@pytest.fixture(scope="module")
def inputs(orc):
    # the draws of make_golden.compute(), in its order
    rng = np.random.default_rng(2024)
    d = {}
    d["x"] = rng.random(37, dtype=np.float32)
    d["xi"] = rng.integers(-1000, 1001, 41, dtype=np.int32)
    d["A"] = rng.standard_normal((6, 5), dtype=np.float32)
    d["y"], d["w"] = rng.standard_normal(37, dtype=np.float32), rng.standard_normal(37, dtype=np.float32)
    d["r"], d["c"] = rng.random((1, 5), dtype=np.float32), rng.random((6, 1), dtype=np.float32)
    d["vr"] = orc.config_inputs("volumerhs", scale=1 / 4000)
    return d


def test_reductions(rk, golden, inputs):
    np.testing.assert_allclose(rk.sum(rk.ROCArray(inputs["x"])), golden["sum_f32"], rtol=1e-5)
    assert int(rk.sum(rk.ROCArray(inputs["xi"]))) == golden["sum_i32"]
    dA = rk.ROCArray(inputs["A"])
    np.testing.assert_allclose(rk.Array(rk.mapreduce(rk.abs2, rk.add, dA, dims=1)).ravel(), golden["abs2sum_dims1"], rtol=1e-5)
    np.testing.assert_allclose(rk.Array(rk.mapreduce(rk.abs2, rk.add, dA, dims=2)).ravel(), golden["abs2sum_dims2"], rtol=1e-5)
    v, i = rk.findmax(dA, dims=1)
    assert np.array_equal(rk.Array(v).ravel(), np.array(golden["findmax_dims1_vals"], dtype=np.float32))
    assert np.array_equal(np.moveaxis(rk.Array(i), 0, -1).reshape(-1), np.array(golden["findmax_dims1_idx"], dtype=np.int64))


def test_scans(rk, golden, inputs):
    assert np.array_equal(rk.Array(rk.cumsum(rk.ROCArray(inputs["xi"]))), np.array(golden["cumsum_i32"], dtype=np.int32))
    got = rk.Array(rk.cumsum(rk.ROCArray(inputs["A"]), dims=1)).reshape(-1, order="F")
    np.testing.assert_allclose(got, golden["cumsum_f32_dims1"], rtol=1e-4)


def test_broadcasts(rk, golden, inputs):
    x, y, w = inputs["x"], inputs["y"], inputs["w"]
    z = rk.ROCArray(dims=x.shape, dtype=np.float32)
    rk.materialize_(z, np.float32(0.5) * rk.lazy(rk.ROCArray(x)) + rk.lazy(rk.ROCArray(y)) * rk.broadcast.exp(rk.lazy(rk.ROCArray(w))))
    ref = np.array(golden["bcast_axpby_exp"])
    bound = 1e-6 * (np.abs(0.5 * x.astype(np.float64)) + np.abs(y.astype(np.float64) * np.exp(w.astype(np.float64)))) + 1e-5 * np.abs(ref)
    assert np.all(np.abs(rk.Array(z) - ref) <= bound)
    A = inputs["A"]
    C = rk.ROCArray(dims=A.shape, dtype=np.float32)
    rk.materialize_(C, rk.lazy(rk.ROCArray(A)) + rk.lazy(rk.ROCArray(inputs["r"])) * rk.lazy(rk.ROCArray(inputs["c"])))
    ref = np.array(golden["bcast_rowcol"], dtype=np.float64)
    np.testing.assert_allclose(rk.Array(C).reshape(-1, order="F"), ref, rtol=1e-6, atol=1e-7)
    host32 = A + inputs["r"].astype(np.float32) * inputs["c"].astype(np.float32)       # separate multiply and add, as Julia evaluates it
    assert host32.dtype == np.float32 and np.array_equal(rk.Array(C), host32)


def test_volumerhs(rk, golden, inputs):
    c = inputs["vr"]
    rhs = rk.ROCArray(c["rhs"])
    rk.volumerhs_(rhs, rk.ROCArray(c["Q"]), rk.ROCArray(c["vgeo"]), c["gravity"], rk.ROCArray(c["D"]), c["Q"].shape[4])
    ref = np.array(golden["volumerhs_1elem"])
    # the same bar as tests/test_volumerhs_gpu.py: rtol 1e-4 plus 2e-6 of the largest entry (ten times the measured error)
    np.testing.assert_allclose(rk.Array(rhs).reshape(-1, order="F"), ref, rtol=1e-4, atol=2e-6 * np.abs(ref).max())
