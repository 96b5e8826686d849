"""Whole configurations on the host checker alone (no GPU): BASELINE's first configuration and the
reference's own default experiment, end to end -- fp16 rounding, norm maps, gate, gated product,
error against the exact fp64 product of the same fp16 operands next to the tau-derived bound."""
import numpy as np

EPS32 = float(np.finfo(np.float32).eps)


def _end_to_end(orc, A, B, tile, tau):
    ref = orc.spamm(A, B, tile, tau)
    nb = A.shape[0] // tile
    dense = orc.gemm_dense_f64(ref["Af"], ref["Bf"])
    err, dn, _ = orc.frob_diff(ref["C"], dense)
    bound = orc.dropped_bound(ref["nA"], ref["nB"], tau)
    floor = EPS32 * np.sqrt(A.shape[1]) * dn          # fp32 accumulation noise, present at tau = 0 too
    # what the gate kept is what a plain restatement of the test keeps
    keep = (ref["nA"][:, None, :] * ref["nB"].T[None, :, :]) >= np.float32(tau)        # [i, j, k], fp32 product
    assert int(keep.sum()) == ref["kept"]
    assert np.array_equal(keep.sum(axis=2).astype(np.int32), ref["counts"])
    # the per-tile bounds hold tile by tile, not only in total
    tiles = orc.dropped_bound_tiles(ref["nA"], ref["nB"], tau)
    diff = (ref["C"].astype(np.float64) - dense).reshape(nb, tile, nb, tile).transpose(0, 2, 1, 3)
    tile_err = np.sqrt((diff ** 2).sum(axis=(2, 3)))
    dtile = np.sqrt((dense.reshape(nb, tile, nb, tile).transpose(0, 2, 1, 3) ** 2).sum(axis=(2, 3)))
    assert np.all(tile_err <= tiles * (1 + 1e-6) + EPS32 * np.sqrt(A.shape[1]) * dtile + 1e-30)
    return ref, err, dn, bound, floor


def test_baseline_config1_on_the_checker(orc):
    # N = 1024, A = B, a_ij = u_ij exp(-0.5 |i-j|), tile 32, tau = 1e-4
    n, b, tau = 1024, 32, 1e-4
    A = orc.fill_decay(n, n, orc.decay_table("exp", n, 0.5), 1)
    ref, err, dn, bound, floor = _end_to_end(orc, A, A.copy(), b, tau)
    frac = ref["kept"] / (n // b) ** 3
    assert 0.007 < frac < 0.010, frac              # ~0.85 % of the 32768 tile products
    assert err <= bound + floor
    assert bound <= tau * (n // b) * (n // b)      # every dropped product is below tau: at most nbK of them per tile
    assert err / dn < 1e-3
    # only the three central diagonals of tiles can be kept: exp(-0.5 d) is gone within one tile
    i, j = np.nonzero(ref["counts"])
    assert np.abs(i - j).max() <= 2


def test_reference_default_experiment_on_the_checker(orc):
    # para.h:1-14 and cuSpAMM.cu:428-431: 2048^3, tile 32 (main.h:32), getDecayMatrixAlg(0.1, 0.1) for
    # both operands (deterministic, no random sign), Norm = 1.548969, fp16 inputs
    n, b, tau = 2048, 32, 1.548969
    tab = orc.decay_table("ref_alg", n, c=0.1, v=0.1)
    assert tab[0] == np.float32(0.1) and tab[1] == np.float32(0.05)       # 0.1 / (0 + 1), 0.1 / (1 + 1)
    A = orc.fill_decay(n, n, tab, 0, random=False)
    assert np.array_equal(A, A.T) and np.array_equal(A[0], tab)          # a function of |i - j| only
    ref, err, dn, bound, floor = _end_to_end(orc, A, A.copy(), b, tau)
    nb = n // b
    frac = ref["kept"] / nb ** 3
    assert 0.04 < frac < 0.06, frac                # the default tau keeps ~4.9 %
    assert err <= bound + floor
    # every tile norm lies between 32 * min|a| and 32 * max|a| of the fp16-rounded table
    assert 32 * 0.1 / (2047 ** 0.1 + 1) * 0.999 < ref["nA"].min() and ref["nA"].max() < 32 * 0.1
    # symmetric input: the norm map of A in role B is the transpose of its map in role A, and the
    # kept set is symmetric under (i, j) -> (j, i)
    assert np.array_equal(ref["nB"], ref["nA"].T)
    assert np.array_equal(ref["counts"], ref["counts"].T)
