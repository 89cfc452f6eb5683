"""GPU parity of volumerhs! against the Float64 oracle (rtol 1e-4, and 2e-6 of the largest entry for entries that
cancel), through the C ABI.  Both kernels are covered: RK_VOLUMERHS_VEC_MIN decides which one a size takes.  The reference has no test for this kernel (perf/ only); the oracle is pinned in
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
    # rtol 1e-4 as the baseline states, plus an absolute term for entries that are differences of large terms.
    # Measured at the baseline configuration (4000 elements): largest error 2.0e-7 of the largest entry; relative error
    # 4e-7 for entries above a tenth of it, 2e-5 above a thousandth.  The absolute term is ten times the measured one.
    scale = np.abs(ref).max()
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=2e-6 * scale)


@pytest.mark.parametrize("nelem", [1, 2, 3, 4, 5, 6, 7, 8, 9, 64, 1001, 1002, 1003])
def test_small(rk, orc, nelem):
    c = orc.config_inputs("volumerhs", scale=nelem / 4000)
    assert c["Q"].shape[4] == nelem
    _close(_run(rk, c), orc.volumerhs(c["rhs"], c["Q"], c["vgeo"], c["gravity"], c["D"]))


def test_four_element_kernel(rk, orc):
    # sizes above the switch-over (32768 elements by default) take the kernel with 16-byte accesses; the remainder of
    # 1, 2 or 3 elements the lane-per-node kernel
    for nelem in (32768, 32771, 40001):
        c = orc.config_inputs("volumerhs", scale=nelem / 4000)
        c["rhs"] = np.random.default_rng(nelem).standard_normal(c["rhs"].shape).astype(np.float32)
        assert c["Q"].shape[4] == nelem
        _close(_run(rk, c), orc.volumerhs(c["rhs"], c["Q"], c["vgeo"], c["gravity"], c["D"]))


def test_config5_full_size(rk, orc):
    c = orc.config_inputs("volumerhs")
    _close(_run(rk, c), orc.volumerhs(c["rhs"], c["Q"], c["vgeo"], c["gravity"], c["D"]))


def test_unaligned_arrays_take_the_scalar_kernel(rk, orc):
    # arrays that start 4 bytes off a 16-byte boundary (views into larger buffers): no 16-byte accesses possible
    nelem = 32770                  # large enough for the four-element kernel, were the arrays aligned
    c = orc.config_inputs("volumerhs", scale=nelem / 4000)
    c["rhs"] = np.random.default_rng(8).standard_normal(c["rhs"].shape).astype(np.float32)

    def shifted(h):
        flat = h.reshape(-1, order="F")
        big = rk.ROCArray(np.concatenate([np.zeros(1, np.float32), flat]))
        return rk.ROCArray(buf=big.buf, dims=h.shape, dtype=np.float32, offset=4)
    rhs = shifted(c["rhs"])
    rk.volumerhs_(rhs, shifted(c["Q"]), shifted(c["vgeo"]), c["gravity"], rk.ROCArray(c["D"]), nelem)
    _close(rk.Array(rhs), orc.volumerhs(c["rhs"], c["Q"], c["vgeo"], c["gravity"], c["D"]))


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
