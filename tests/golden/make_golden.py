"""Writes tests/golden/oracle_golden.json: small, seeded input -> output vectors of the NumPy oracle.

    python -m tests.golden.make_golden

The reference tree has no golden vectors for this path and cannot be executed here (it is Julia; no
runtime on this machine), so these fixtures record the oracle's own answers on tiny seeded cases.  They
guard the oracle against silent drift; what makes the oracle *right* is checked in tests/test_oracle.py."""
import json
import os

import numpy as np

from oracle import oracle as orc


def compute():
    rng = np.random.default_rng(2024)
    out = {}
    x = rng.random(37, dtype=np.float32)
    xi = rng.integers(-1000, 1001, 41, dtype=np.int32)
    A = rng.standard_normal((6, 5), dtype=np.float32)
    out["sum_f32"] = float(orc.sum_(x))
    out["sum_i32"] = int(orc.sum_(xi))
    out["abs2sum_dims1"] = orc.mapreduce("abs2", "add", A, dims=1).ravel().tolist()
    out["abs2sum_dims2"] = orc.mapreduce("abs2", "add", A, dims=2).ravel().tolist()
    v, i = orc.findmax(A, dims=1)
    out["findmax_dims1_vals"] = v.ravel().tolist()
    out["findmax_dims1_idx"] = i.reshape(-1).tolist()
    out["cumsum_i32"] = orc.cumsum(xi).tolist()
    out["cumsum_f32_dims1"] = orc.cumsum(A, dims=1).reshape(-1, order="F").tolist()
    y, w = rng.standard_normal(37, dtype=np.float32), rng.standard_normal(37, dtype=np.float32)
    out["bcast_axpby_exp"] = orc.broadcast_axpby_exp(np.float32(0.5), x, y, w).tolist()
    r, c = rng.random((1, 5), dtype=np.float32), rng.random((6, 1), dtype=np.float32)
    out["bcast_rowcol"] = orc.broadcast_rowcol(A, r, c).reshape(-1, order="F").tolist()
    cfg = orc.config_inputs("volumerhs", scale=1 / 4000)
    out["volumerhs_1elem"] = orc.volumerhs(cfg["rhs"], cfg["Q"], cfg["vgeo"], cfg["gravity"], cfg["D"]).reshape(-1, order="F").tolist()
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_golden.json")
    with open(path, "w") as fh:
        json.dump(compute(), fh)
    print("wrote", path)
