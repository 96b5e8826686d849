"""Pins the checker's tau gate (cuSpAMM.cu:303-311 fp32 product >= tau,
:315-325 ascending compaction, :328-334 count; tool.cu:493-529 kept count)."""
import numpy as np


def _maps(rng, nbM, nbK, nbN):
    nA = np.abs(rng.normal(size=(nbM, nbK))).astype(np.float32)
    nB = np.abs(rng.normal(size=(nbK, nbN))).astype(np.float32)
    return nA, nB


def _numpy_keep(nA, nB, tau):
    # countValid (tool.cu:505-516): norm = nA[i,k]*nB[k,j] in float; keep iff norm >= tau
    p = nA[:, None, :] * nB.T[None, :, :]                   # [i, j, k], fp32 products
    assert p.dtype == np.float32
    return p >= np.float32(tau)


def _unpack(mask, nbK):
    bits = np.unpackbits(mask.view(np.uint8), axis=-1, bitorder="little")
    return bits[..., :nbK].astype(bool)


def test_tau_zero_keeps_everything_and_inf_nothing(orc):
    rng = np.random.default_rng(0)
    nA, nB = _maps(rng, 5, 70, 3)
    nA[2, 7] = 0.0                                           # 0*x >= 0 still kept
    total, counts, klist, mask = orc.gate(nA, nB, 0.0)
    assert total == 5 * 70 * 3 and np.all(counts == 70)
    assert np.all(klist == np.arange(70, dtype=np.uint16))
    total, counts, klist, mask = orc.gate(nA, nB, np.inf)
    assert total == 0 and np.all(counts == 0) and np.all(mask == 0)


def test_matches_numpy_restatement_of_count_valid(orc):
    rng = np.random.default_rng(1)
    for nbM, nbK, nbN in [(4, 64, 4), (3, 65, 5), (7, 130, 2), (1, 1, 1)]:
        nA, nB = _maps(rng, nbM, nbK, nbN)
        for tau in (0.05, 0.5, 1.5):
            keep = _numpy_keep(nA, nB, tau)
            total, counts, klist, mask = orc.gate(nA, nB, tau)
            assert total == int(keep.sum())
            assert np.array_equal(counts, keep.sum(axis=2))
            assert np.array_equal(_unpack(mask, nbK), keep)
            for i in range(nbM):
                for j in range(nbN):
                    assert np.array_equal(klist[i, j, :counts[i, j]], np.nonzero(keep[i, j])[0])


def test_exact_equality_is_kept(orc):
    # pins '>=' (cuSpAMM.cu:306) against '>' (cuSpAMM.cu:150): 2*3 == 6 exactly
    nA = np.array([[2.0, 1.0], [0.5, 4.0]], dtype=np.float32)
    nB = np.array([[3.0, 1.0], [6.0, 1.5]], dtype=np.float32)
    total, counts, klist, mask = orc.gate(nA, nB, 6.0)
    # products: (0,0): k0 6 keep, k1 6 keep ; (0,1): 2, 1.5 ; (1,0): 1.5, 24 keep ; (1,1): .5, 6 keep
    assert counts.tolist() == [[2, 0], [1, 1]]
    assert klist[1, 0, 0] == 1 and klist[1, 1, 0] == 1
    above = np.nextafter(np.float32(6.0), np.float32(7.0))
    total2, counts2, _, _ = orc.gate(nA, nB, above)
    assert counts2.tolist() == [[0, 0], [1, 0]]


def test_product_is_rounded_to_fp32_before_compare(orc):
    # find a*b whose fp32 rounding goes UP: with tau = fl32(a*b) the fp32 gate keeps the product
    # (cuSpAMM.cu:305-306 multiplies and compares floats) while a double-precision compare of
    # the exact product would drop it.
    rng = np.random.default_rng(5)
    found = 0
    for _ in range(200):
        a = np.float32(rng.uniform(1, 2))
        b = np.float32(rng.uniform(1, 2))
        p32 = np.float32(a * b)
        exact = float(a) * float(b)                          # exact in double (24+24 bits)
        if float(p32) > exact:
            nA = np.array([[a]], dtype=np.float32)
            nB = np.array([[b]], dtype=np.float32)
            assert orc.gate(nA, nB, p32)[0] == 1
            assert orc.gate(nA, nB, np.nextafter(p32, np.float32(4)))[0] == 0
            found += 1
    assert found > 20


def test_monotone_in_tau(orc):
    rng = np.random.default_rng(2)
    nA, nB = _maps(rng, 6, 40, 6)
    prev = None
    for tau in (0.0, 0.01, 0.1, 0.5, 1.0, 3.0, 100.0):
        _, _, _, mask = orc.gate(nA, nB, tau)
        keep = _unpack(mask, 40)
        if prev is not None:
            assert not np.any(keep & ~prev)
        prev = keep


def test_tau_for_ratio_and_bisection(orc):
    rng = np.random.default_rng(3)
    nA, nB = _maps(rng, 8, 32, 8)
    for ratio in (0.05, 0.2, 0.5, 0.75):
        tau, ach = orc.tau_for_ratio(nA, nB, ratio)
        total, *_ = orc.gate(nA, nB, tau)
        n = 8 * 32 * 8
        assert total == round(ach * n)
        assert total >= int(np.ceil(ratio * n)) and total <= int(np.ceil(ratio * n)) + 1
        up = np.nextafter(np.float32(tau), np.float32(np.inf))
        assert orc.gate(nA, nB, up)[0] < int(np.ceil(ratio * n))
    # tuneValidRate (tool.cu:438-490): within +-1% of 75% after at most 20 rounds on a smooth map
    tau, ach = orc.tune_bisect(nA, nB, 0.75, 0.01, 20)
    assert abs(ach - 0.75) < 0.01
    assert abs(orc.gate(nA, nB, tau)[0] / (8 * 32 * 8) - ach) < 1e-6


def test_zero_tail_gives_smallest_positive_tau(orc):
    nA = np.array([[1.0, 0.0, 0.0, 0.0]], dtype=np.float32)
    nB = np.ones((4, 1), dtype=np.float32)
    tau, ach = orc.tau_for_ratio(nA, nB, 0.5)               # only 25 % reachable with tau > 0
    assert tau == 1.0 and ach == 0.25
