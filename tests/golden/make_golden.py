"""Writes tests/golden/penc_golden.npz: small seeded cases (one per pos_dim 2..8) with the CPU
oracle's outputs, so that (a) a later change of the oracle that alters results is noticed and
(b) the GPU path can be checked against fixed vectors without rebuilding anything.

The reference itself ships no vectors and cannot run here (CUDA-only), so these are produced by
the oracle, which is pinned independently by tests/test_oracle_pinning.py.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import api as orc  # noqa: E402

N, LEVELS, CAP = 96, 5, 256


def make_case(d):
    rng = np.random.default_rng(1000 + d)
    sigmas = np.geomspace(1.0, 5e-3, LEVELS).astype(np.float32)
    c = dict(
        sigmas=sigmas,
        pos=rng.uniform(0, 1, (N, d)).astype(np.float32),
        shift=(rng.standard_normal((LEVELS, d)) * 10).astype(np.float32),
        table=rng.uniform(-1, 1, (LEVELS, CAP, 2)).astype(np.float32),
        window=np.array([1.0, 0.75, 1.0, 0.0, 0.5], np.float32),
        grad=rng.standard_normal((LEVELS, 2, N)).astype(np.float32),
        dpos=rng.standard_normal((N, d)).astype(np.float32),
    )
    sf = orc.scale_factors(d, sigmas)
    s = orc.simplex(c["pos"], sf, c["shift"], CAP)
    c.update(sf=sf, rem0=s["rem0"], rank=s["rank"], slot=s["slot"], bary=s["bary"])
    c["out"] = orc.forward(c["pos"], c["table"], sf, c["shift"], c["window"])
    c["table_grad"] = orc.backward_table(c["pos"], sf, c["shift"], c["window"], c["grad"], CAP)["grad64"]
    c["pos_grad"] = orc.backward_pos(c["pos"], c["table"], sf, c["shift"], c["window"], c["grad"])["grad64"]
    r = orc.double_backward(c["pos"], c["table"], sf, c["shift"], c["window"], c["dpos"], c["grad"])
    c["table_grad2"] = r["grad64"]
    c["ggs"] = r["ggs"]
    return c


if __name__ == "__main__":
    out = {}
    for d in range(2, 9):
        for k, v in make_case(d).items():
            out[f"d{d}_{k}"] = v
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "penc_golden.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")
