"""Pins the checker's gated tile product (cuSpAMM.cu:358-375: sum over kept k
of A_ik * B_kj, fp16 operands, fp32 accumulate; :391 row-major C)."""
import numpy as np
import pytest


def _inputs(orc, M, K, N, lam, seedA=1, seedB=2):
    tab = orc.decay_table("exp", max(M, K, N), lam)
    return orc.fill_decay(M, K, tab, seedA), orc.fill_decay(K, N, tab, seedB)


@pytest.mark.parametrize("b", [32, 64, 128])
def test_tau_zero_equals_dense_gemm(orc, b):
    A, B = _inputs(orc, 2 * b, 3 * b, 4 * b, 0.01)
    r = orc.spamm(A, B, b, 0.0)
    assert r["kept"] == 2 * 3 * 4
    dense = r["Af"].astype(np.float64) @ r["Bf"].astype(np.float64)
    err = np.linalg.norm(r["C"] - dense) / np.linalg.norm(dense)
    assert err < 2e-6                                        # fp32 accumulation only
    # the checker's own fp64 dense product agrees with numpy's
    Cd = orc.gemm_dense_f64(r["Af"], r["Bf"])
    assert np.allclose(Cd, dense, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("b", [32, 64])
def test_all_ones_gives_k_exactly(orc, b):
    A = np.ones((2 * b, 5 * b), dtype=np.float32)
    B = np.ones((5 * b, 3 * b), dtype=np.float32)
    r = orc.spamm(A, B, b, 0.0)
    assert np.all(r["C"] == 5 * b)
    # tile norm products are b*b; tau above that drops everything
    r = orc.spamm(A, B, b, float(b * b) + 1.0)
    assert r["kept"] == 0 and np.all(r["C"] == 0)
    r = orc.spamm(A, B, b, float(b * b))
    assert r["kept"] == 2 * 5 * 3 and np.all(r["C"] == 5 * b)


def test_identity_copies_kept_tiles_of_b(orc):
    b, n = 32, 128
    _, B = _inputs(orc, n, n, n, 0.05)
    A = np.eye(n, dtype=np.float32)
    tau = 10.0
    r = orc.spamm(A, B, b, tau)
    keep = (np.sqrt(np.float32(b)) * r["nB"]) >= np.float32(tau)      # ||I_tile|| = sqrt(b); k must equal i
    expect = np.zeros_like(B)
    for i in range(n // b):
        for j in range(n // b):
            if keep[i, j]:
                expect[i * b:(i + 1) * b, j * b:(j + 1) * b] = r["Bf"][i * b:(i + 1) * b, j * b:(j + 1) * b]
    assert 0 < keep.sum() < keep.size
    assert np.array_equal(r["C"], expect)


def test_block_diagonal_stays_block_diagonal(orc):
    b, n = 32, 128
    A, B = _inputs(orc, n, n, n, 0.0)
    blk = np.kron(np.eye(2), np.ones((2 * b, 2 * b))).astype(np.float32)
    A *= blk
    B *= blk
    r = orc.spamm(A, B, b, 1e-3)
    assert np.all(r["C"][blk == 0] == 0)
    dense = (r["Af"].astype(np.float64) @ r["Bf"].astype(np.float64))
    assert np.linalg.norm(r["C"] - dense) / np.linalg.norm(dense) < 2e-6
    assert r["kept"] == 2 * (2 * 2 * 2)                      # zero tiles have norm 0 < tau


def test_brute_force_tiny(orc):
    # plain loops over (i, j, k) tiles with an independently evaluated mask
    b = 32
    A, B = _inputs(orc, 2 * b, 3 * b, 2 * b, 0.08)
    tau = 0.8
    r = orc.spamm(A, B, b, tau)
    Af = A.astype(np.float16).astype(np.float64)
    Bf = B.astype(np.float16).astype(np.float64)
    C = np.zeros((2 * b, 2 * b))
    kept = 0
    for i in range(2):
        for j in range(2):
            for k in range(3):
                ta = Af[i * b:(i + 1) * b, k * b:(k + 1) * b]
                tb = Bf[k * b:(k + 1) * b, j * b:(j + 1) * b]
                na = np.float32(np.sqrt((ta ** 2).sum()))
                nb_ = np.float32(np.sqrt((tb ** 2).sum()))
                if np.float32(na * nb_) >= np.float32(tau):
                    C[i * b:(i + 1) * b, j * b:(j + 1) * b] += ta @ tb
                    kept += 1
    assert 0 < kept < 12
    assert r["kept"] == kept
    assert np.linalg.norm(r["C"] - C) / np.linalg.norm(C) < 2e-6


def test_dropped_norm_bound(orc):
    # ||C_spamm - C_exact||_F <= sqrt(sum_ij (sum_{k dropped} nA_ik nB_kj)^2)
    b, n = 32, 512
    A, B = _inputs(orc, n, n, n, 0.02)
    for tau in (1e-3, 1e-1, 1.0, 5.0):
        r = orc.spamm(A, B, b, tau)
        dense = orc.gemm_dense_f64(r["Af"], r["Bf"])
        err, dn, _ = orc.frob_diff(r["C"], dense)
        bound = orc.dropped_bound(r["nA"], r["nB"], tau)
        nb = n // b
        assert err <= bound * (1 + 1e-5) + 1e-5 * dn
        assert bound <= tau * nb * np.sqrt(nb * nb) * (1 + 1e-6)
    assert 0 < r["kept"] < nb ** 3


def test_dropped_bound_hand_worked(orc):
    # nA = [[1,2,3],[4,5,6]], nB = [[1,2],[3,4],[5,6]]; products per output tile (k = 0,1,2):
    #   (0,0): 1, 6, 15   (0,1): 2, 8, 18   (1,0): 4, 15, 30   (1,1): 8, 20, 36
    # tau = 10 drops everything below 10: sums 7, 10, 4, 8 -> sqrt(49 + 100 + 16 + 64) = sqrt(229)
    # tau = 8 keeps the two products equal to 8 (>=): sums 7, 2, 4, 0 -> sqrt(69)
    nA = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.float32)
    nB = np.array([[1, 2], [3, 4], [5, 6]], dtype=np.float32)
    assert orc.dropped_bound(nA, nB, 10.0) == pytest.approx(np.sqrt(229.0), rel=1e-15)
    assert orc.dropped_bound(nA, nB, 8.0) == pytest.approx(np.sqrt(69.0), rel=1e-15)
    assert orc.dropped_bound(nA, nB, 10.0, 1, 2) == pytest.approx(np.sqrt(80.0), rel=1e-15)      # tile row 1 only
    assert orc.dropped_bound(nA, nB, 0.0) == 0.0                                                  # nothing dropped
    assert orc.dropped_bound(nA, nB, 37.0) == pytest.approx(np.sqrt(22.0 ** 2 + 28.0 ** 2 + 49.0 ** 2 + 64.0 ** 2), rel=1e-15)
    # the product that is compared is the fp32 one: 3 * (1/3 rounded) is exactly 1 in fp32, so it is
    # kept at tau = 1 although the exact product of the two floats lies just above or below 1
    third = np.float32(1.0) / np.float32(3.0)
    assert np.float32(3.0) * third == np.float32(1.0)
    assert orc.dropped_bound(np.array([[3.0]], dtype=np.float32), np.array([[third]], dtype=np.float32), 1.0) == 0.0


def test_dropped_bound_tiles_hand_worked(orc):
    # same map as above: per-tile dropped sums at tau = 10 are 7, 10 / 4, 8; at tau = 8: 7, 2 / 4, 0
    nA = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.float32)
    nB = np.array([[1, 2], [3, 4], [5, 6]], dtype=np.float32)
    assert np.array_equal(orc.dropped_bound_tiles(nA, nB, 10.0), np.array([[7.0, 10.0], [4.0, 8.0]]))
    assert np.array_equal(orc.dropped_bound_tiles(nA, nB, 8.0), np.array([[7.0, 2.0], [4.0, 0.0]]))
    assert np.array_equal(orc.dropped_bound_tiles(nA, nB, 0.0), np.zeros((2, 2)))
    # everything dropped: the tile sums are the plain product of the norm maps
    assert np.array_equal(orc.dropped_bound_tiles(nA, nB, 1e9), nA.astype(np.float64) @ nB.astype(np.float64))
    # and the scalar bound is the root of the sum of their squares, row range by row range
    rng = np.random.default_rng(5)
    a, b = rng.random((5, 7), dtype=np.float32), rng.random((7, 4), dtype=np.float32)
    t = orc.dropped_bound_tiles(a, b, 0.3)
    assert orc.dropped_bound(a, b, 0.3) == pytest.approx(np.sqrt((t ** 2).sum()), rel=1e-14)
    assert orc.dropped_bound(a, b, 0.3, 2, 4) == pytest.approx(np.sqrt((t[2:4] ** 2).sum()), rel=1e-14)


def test_row_slab_interface(orc):
    b, n = 32, 128
    A, B = _inputs(orc, n, n, n, 0.02)
    r = orc.spamm(A, B, b, 0.1)
    part = orc.gemm_gated(r["Af"], r["Bf"], b, r["counts"], r["klist"], ti0=1, ti1=3)
    assert np.array_equal(part[b:3 * b], r["C"][b:3 * b])
    assert np.all(part[:b] == 0) and np.all(part[3 * b:] == 0)


def test_frob_metrics(orc):
    rng = np.random.default_rng(0)
    X = rng.normal(size=1000).astype(np.float32)
    Y = rng.normal(size=1000)
    e, y, x = orc.frob_diff(X, Y)
    assert np.isclose(e, np.linalg.norm(X - Y)) and np.isclose(y, np.linalg.norm(Y)) and np.isclose(x, np.linalg.norm(X.astype(np.float64)))
