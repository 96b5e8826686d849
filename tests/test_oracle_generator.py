"""Pins the seeded u_ij * decay(|i-j|) generator (tool.cu:409-436 family)."""
import numpy as np


def test_uniform_range_and_moments(orc):
    n = 1024
    X = orc.fill_decay(n, n, orc.decay_table("none", n), seed=1)
    assert X.min() >= -1.0 and X.max() < 1.0
    # multiples of 2^-23
    assert np.all(X * 2.0 ** 23 == np.round(X * 2.0 ** 23))
    assert abs(X.mean()) < 3e-3
    assert abs((X.astype(np.float64) ** 2).mean() - 1.0 / 3.0) < 3e-3
    Y = orc.fill_decay(n, n, orc.decay_table("none", n), seed=2)
    assert abs(np.corrcoef(X.ravel(), Y.ravel())[0, 1]) < 5e-3
    # neighbouring entries are uncorrelated
    assert abs(np.corrcoef(X[:, :-1].ravel(), X[:, 1:].ravel())[0, 1]) < 5e-3


def test_decay_factorisation(orc):
    n = 256
    tab = orc.decay_table("exp", n, 0.1)
    U = orc.fill_decay(n, n, orc.decay_table("none", n), seed=5)
    X = orc.fill_decay(n, n, tab, seed=5)
    i, j = np.indices((n, n))
    assert np.array_equal(X, U * tab[np.abs(i - j)])     # one fp32 multiply, exact


def test_rectangular_index(orc):
    # element (i,j) depends on the linear index i*cols+j of ITS matrix
    tab = orc.decay_table("none", 512)
    X = orc.fill_decay(64, 512, tab, seed=9)
    Y = orc.fill_decay(128, 256, tab, seed=9)
    assert np.array_equal(X.ravel()[:4096], Y.ravel()[:4096])


def test_reference_generators(orc):
    # tool.cu:409-422: c * v^|i-j| ; tool.cu:426-436: c / (|i-j|^v + 1); deterministic (random=0)
    n = 128
    i, j = np.indices((n, n))
    d = np.abs(i - j)
    E = orc.fill_decay(n, n, orc.decay_table("ref_exp", n, c=1.0, v=0.1), seed=0, random=False)
    ref = (np.float32(1.0) * np.power(np.float64(np.float32(0.1)), d).astype(np.float32))
    assert np.array_equal(E, ref.astype(np.float32))
    A = orc.fill_decay(n, n, orc.decay_table("ref_alg", n, c=0.1, v=0.1), seed=0, random=False)
    ref = np.float32(0.1) / (np.power(d.astype(np.float64), np.float64(np.float32(0.1))).astype(np.float32) + np.float32(1))
    assert np.array_equal(A, ref.astype(np.float32))
    assert A[0, 0] == np.float32(0.1)       # d = 0 -> c / (0 + 1)
    O = orc.fill_decay(n, n, orc.decay_table("none", n), seed=0, random=False)
    assert np.all(O == 1.0)                 # getNormMatrix, tool.cu:370-403
