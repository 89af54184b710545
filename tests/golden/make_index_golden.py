"""Writes tests/golden/index_calc_golden.npz from the REFERENCE's own index_calculation.

The reference translation unit inference-engine/src/host/index_calc_host.cpp is compiled from
source by oracle/Makefile into oracle/_ref/libref_index_calc.so (this only works in a container
that holds the reference tree).  This script feeds it small seeded inputs and records inputs and
outputs; the fixture is data only.  Run from the repo root:

    make -C oracle && python tests/golden/make_index_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402


def near_tie_case(rng, N, CB, C, v):
    """Inputs that sit (almost) midway between centroids, so that many distance pairs differ by
    about 1e-6 and the scan's hysteresis matters."""
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    x = np.empty((N, CB * v), dtype=np.float32)
    for n in range(N):
        for cb in range(CB):
            a, b = rng.choice(C, size=2, replace=False)
            mid = (cent[cb, a] + cent[cb, b]) * np.float32(0.5)
            x[n, cb * v:(cb + 1) * v] = mid + rng.standard_normal(v).astype(np.float32) * np.float32(2e-7)
    return x, cent


def main():
    assert oracle.have_ref(), "build oracle/_ref first (needs the reference tree)"
    rng = np.random.default_rng(20240427)
    out = {}
    cases = []
    cid = 0
    for v in (2, 4, 8):
        for C in (8, 16, 32):
            N, CB = 12, 6
            x = rng.standard_normal((N, CB * v)).astype(np.float32)
            cent = rng.standard_normal((CB, C, v)).astype(np.float32)
            cases.append(("randn", x, cent, v, N, CB))
            xt, ct = near_tie_case(rng, N, CB, C, v)
            cases.append(("neartie", xt, ct, v, N, CB))
    # the reference test driver's own value ranges (test_amm.cpp:26-45): U(-5,5), U(-10,10)
    for v, C in ((4, 16), (2, 16)):
        N, CB = 16, 8
        x = rng.uniform(-5, 5, (N, CB * v)).astype(np.float32)
        cent = rng.uniform(-10, 10, (CB, C, v)).astype(np.float32)
        cases.append(("uniform", x, cent, v, N, CB))
    # duplicated centroids: exact ties must keep the earlier index
    v, C, N, CB = 4, 16, 8, 4
    cent = rng.standard_normal((CB, C, v)).astype(np.float32)
    cent[:, 8:] = cent[:, :8]
    x = rng.standard_normal((N, CB * v)).astype(np.float32)
    cases.append(("dupcent", x, cent, v, N, CB))

    for kind, x, cent, v, N, CB in cases:
        idx = oracle.ref_index_calculation(x, cent, v)
        out[f"c{cid}_kind"] = np.array(kind)
        out[f"c{cid}_x"] = x
        out[f"c{cid}_cent"] = cent
        out[f"c{cid}_idx"] = idx
        # one non-identity tiling per case (index_calc_host.cpp:41-49)
        n_stile, cb_mtile = N // 2, CB // 2
        out[f"c{cid}_tiled_{n_stile}_{cb_mtile}"] = oracle.ref_index_calculation(x, cent, v, n_stile, cb_mtile)
        cid += 1
    out["ncases"] = np.array(cid)
    path = os.path.join(ROOT, "tests", "golden", "index_calc_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, "cases:", cid, "bytes:", os.path.getsize(path))


if __name__ == "__main__":
    main()
