"""GPU parity of volumerhs! against the Float64 oracle (rtol 1e-4 of the element-wise scale), through
the C ABI.  The reference has no test for this kernel (perf/ only); the oracle is pinned in
tests/test_oracle.py."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run(rk, c):
    rhs = rk.ROCArray(c["rhs"])
    out = rk.volumerhs_(rhs, rk.ROCArray(c["Q"]), rk.ROCArray(c["vgeo"]), c["gravity"], rk.ROCArray(c["D"]), c["Q"].shape[4])
    assert out is rhs
    return rk.Array(rhs)


def _close(got, ref):
    # rtol 1e-4 relative to the magnitude of the sums that form each entry (cancellation-safe)
    scale = np.abs(ref).max()
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-4 * scale)


@pytest.mark.parametrize("nelem", [1, 2, 3, 7, 64, 1001])
def test_small(rk, orc, nelem):
    c = orc.config_inputs("volumerhs", scale=nelem / 4000)
    assert c["Q"].shape[4] == nelem
    _close(_run(rk, c), orc.volumerhs(c["rhs"], c["Q"], c["vgeo"], c["gravity"], c["D"]))


def test_config5_full_size(rk, orc):
    c = orc.config_inputs("volumerhs")
    _close(_run(rk, c), orc.volumerhs(c["rhs"], c["Q"], c["vgeo"], c["gravity"], c["D"]))


def test_accumulates_into_rhs(rk, orc):
    c = orc.config_inputs("volumerhs", scale=10 / 4000)
    c["rhs"] = np.random.default_rng(5).standard_normal(c["rhs"].shape).astype(np.float32)
    _close(_run(rk, c), orc.volumerhs(c["rhs"], c["Q"], c["vgeo"], c["gravity"], c["D"]))


def test_reference_harness_inputs(rk, orc):
    # value ranges of perf/volumerhs.jl:187-195: Q = 1 + rand, E += 20, MJ = rand + 3, MJI = 1 / MJ
    rng = np.random.default_rng(123)
    ne = 50
    Q = (1 + rng.random((5, 5, 5, 5, ne))).astype(np.float32)
    Q[:, :, :, 4, :] += 20
    vgeo = rng.random((5, 5, 5, 14, ne)).astype(np.float32)
    vgeo[:, :, :, 9, :] += 3
    vgeo[:, :, :, 10, :] = 1 / vgeo[:, :, :, 9, :]
    D = rng.random((5, 5)).astype(np.float32)
    c = {"Q": Q, "vgeo": vgeo, "D": D, "gravity": np.float32(9.81), "rhs": np.zeros_like(Q)}
    _close(_run(rk, c), orc.volumerhs(c["rhs"], Q, vgeo, c["gravity"], D))


def test_constant_state_invariant(rk):
    # columns of D summing to zero annihilate constants: with constant Q and metrics only -g*rho remains on W
    ne = 5
    Q = np.empty((5, 5, 5, 5, ne), dtype=np.float32)
    for s, v in enumerate((1.2, 0.3, -0.2, 0.1, 25.0)):
        Q[:, :, :, s, :] = v
    vgeo = np.empty((5, 5, 5, 14, ne), dtype=np.float32)
    for f in range(14):
        vgeo[:, :, :, f, :] = 0.9 + 0.01 * f
    vgeo[:, :, :, 10, :] = 1 / vgeo[:, :, :, 9, :]
    D = np.random.default_rng(6).standard_normal((5, 5)).astype(np.float32)
    D -= D.mean(axis=0, keepdims=True)
    c = {"Q": Q, "vgeo": vgeo, "D": D, "gravity": np.float32(9.81), "rhs": np.zeros_like(Q)}
    got = _run(rk, c)
    want = np.zeros_like(Q, dtype=np.float64)
    want[:, :, :, 3, :] = -1.2 * 9.81 * (np.float64(vgeo[0, 0, 0, 9, 0]) * np.float64(vgeo[0, 0, 0, 10, 0]))
    np.testing.assert_allclose(got, want, atol=2e-3)


def test_argument_checks(rk):
    z = rk.zeros(np.float32, 5, 5, 5, 5, 2)
    vg = rk.zeros(np.float32, 5, 5, 5, 14, 2)
    D = rk.zeros(np.float32, 5, 5)
    with pytest.raises(rk.DimensionMismatch):
        rk.volumerhs_(z, z, vg, 9.81, D, 3)
    with pytest.raises(rk.UnsupportedError):
        rk.volumerhs_(rk.zeros(np.float64, 5, 5, 5, 5, 2), z, vg, 9.81, D, 2)
