"""The checker against its own frozen vectors (tests/golden/spamm_small.npz),
so that neither the checker nor the generator can drift unnoticed."""
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
NAMES = ["exp_b32", "exp_b64_rect", "alg_b32", "exp_b128"]


@pytest.fixture(scope="module")
def gold():
    return np.load(os.path.join(HERE, "golden", "spamm_small.npz"))


@pytest.mark.parametrize("name", NAMES)
def test_checker_reproduces_golden(orc, gold, name):
    M, K, N, tile = (int(v) for v in gold[name + "_cfg"])
    tau = float(gold[name + "_tau"][0])
    tab = gold[name + "_table"]
    A = orc.fill_decay(M, K, tab, 1)
    B = orc.fill_decay(K, N, tab, 2)
    assert np.array_equal(A[:4, :8], gold[name + "_A_sample"])
    assert np.array_equal(B[-4:, -8:], gold[name + "_B_sample"])
    r = orc.spamm(A, B, tile, tau)
    assert np.array_equal(r["nA"].view(np.uint32), gold[name + "_nA"].view(np.uint32))
    assert np.array_equal(r["nB"].view(np.uint32), gold[name + "_nB"].view(np.uint32))
    assert np.array_equal(r["counts"], gold[name + "_counts"])
    assert np.array_equal(r["mask"], gold[name + "_mask"])
    assert np.array_equal(r["C"], gold[name + "_C"])
    kept = int(r["counts"].sum())
    assert 0 < kept < r["counts"].size * (K // tile)          # the case exercises the gate
