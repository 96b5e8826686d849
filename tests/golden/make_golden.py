"""Writes tests/golden/spamm_small.npz: frozen input/output vectors of the host
checker for small cases (the reference ships no fixtures of its own).  The
checker is first pinned by the closed-form and brute-force tests in tests/;
these vectors then keep it (and the HIP path) from drifting.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as orc  # noqa: E402

CASES = [
    # name, M, K, N, tile, kind, lam, tau
    ("exp_b32", 128, 128, 128, 32, "exp", 0.05, 0.5),
    ("exp_b64_rect", 128, 192, 256, 64, "exp", 0.02, 100.0),
    ("alg_b32", 160, 96, 128, 32, "alg", 0.0, 1e-3),
    ("exp_b128", 256, 256, 256, 128, "exp", 0.01, 1000.0),
]


def main():
    out = {}
    for name, M, K, N, tile, kind, lam, tau in CASES:
        tab = orc.decay_table(kind, max(M, K, N), lam)
        A = orc.fill_decay(M, K, tab, 1)
        B = orc.fill_decay(K, N, tab, 2)
        r = orc.spamm(A, B, tile, tau)
        out[name + "_table"] = tab
        out[name + "_cfg"] = np.array([M, K, N, tile], dtype=np.int64)
        out[name + "_tau"] = np.array([tau], dtype=np.float32)
        out[name + "_A_sample"] = A[:4, :8].copy()           # spot values of the generator
        out[name + "_B_sample"] = B[-4:, -8:].copy()
        out[name + "_nA"] = r["nA"]
        out[name + "_nB"] = r["nB"]
        out[name + "_counts"] = r["counts"]
        out[name + "_mask"] = r["mask"]
        out[name + "_C"] = r["C"]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "spamm_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path))


if __name__ == "__main__":
    main()
