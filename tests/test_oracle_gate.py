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


# tuneValidRate worked by hand from tool.cu:445-486 on the 1 x 4 x 1 map with products 1, 2, 3, 4
# (kept ratio is a multiple of 1/4, so targets 0.6 and 0.1 are never met and the loop runs until
# max_rounds).  Round 0 measures the ratio at Norm = 0 (1.0) and moves to the mean product 2.5 = up.
#   expected 0.6: 2.5 (ratio .5 < .6: up = 2.5, Norm = (2.5 + 0) / 2)  -> 1.25 (.75 > .6: down = 1.25,
#     Norm = (1.25 + 2.5) / 2) -> 1.875 (.75: down = 1.875) -> 2.1875 (.5: up = 2.1875) -> 2.03125
#     (.5: up) -> 1.953125 (.75: down) -> 1.9921875
#   expected 0.1: 2.5 (.5 > .1 and up == Norm: up = 5, down = 2.5) -> 3.75 (.25 > .1: down = 3.75)
#     -> 4.375 (0 < .1: up = 4.375) -> 4.0625 (0: up) -> 3.90625 (.25: down) -> 3.984375
# The value returned after r rounds is the Norm entering round r; the ratio is the one measured in
# round r - 1.
BISECT_HAND = {
    0.6: [(2.5, 1.0), (1.25, 0.5), (1.875, 0.75), (2.1875, 0.75), (2.03125, 0.5), (1.953125, 0.5), (1.9921875, 0.75)],
    0.1: [(2.5, 1.0), (3.75, 0.5), (4.375, 0.25), (4.0625, 0.0), (3.90625, 0.0), (3.984375, 0.25)],
}


def test_bisection_iterates_match_the_hand_worked_sequence(orc):
    nA = np.array([[1.0, 2.0, 3.0, 4.0]], dtype=np.float32)
    nB = np.ones((4, 1), dtype=np.float32)
    for expected, seq in BISECT_HAND.items():
        for rounds, (norm, rate) in enumerate(seq, start=1):
            tau, ach = orc.tune_bisect(nA, nB, expected, 0.01, rounds)
            assert (tau, ach) == (norm, rate), (expected, rounds, tau, ach)
    # targets that are met stop early: 0.5 after round 1 (Norm 2.5 keeps 3 and 4), 0.25 after the
    # doubling step (3.75 keeps 4), 0.75 after one halving (1.25 keeps 2, 3, 4), 1.0 at once (Norm 0)
    assert orc.tune_bisect(nA, nB, 0.5, 0.01, 20) == (2.5, 0.5)
    assert orc.tune_bisect(nA, nB, 0.25, 0.01, 20) == (3.75, 0.25)
    assert orc.tune_bisect(nA, nB, 0.75, 0.01, 20) == (1.25, 0.75)
    assert orc.tune_bisect(nA, nB, 1.0, 0.01, 20) == (0.0, 1.0)


def test_zero_tail_gives_smallest_positive_tau(orc):
    nA = np.array([[1.0, 0.0, 0.0, 0.0]], dtype=np.float32)
    nB = np.ones((4, 1), dtype=np.float32)
    tau, ach = orc.tau_for_ratio(nA, nB, 0.5)               # only 25 % reachable with tau > 0
    assert tau == 1.0 and ach == 0.25
