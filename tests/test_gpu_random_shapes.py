"""Seeded random shapes, decays, zero blocks and thresholds: every gate output and C against the
checker, and the tau-aware passes against the plain call."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_cases_against_the_checker(orc, ctx, seed):
    import torch
    rng = np.random.default_rng(seed)
    for case in range(10):
        tile = int(rng.choice([32, 64, 128]))
        M, K, N = [int(rng.integers(1, 1 + 1200 // tile)) * tile for _ in range(3)]
        kind = str(rng.choice(["exp", "alg"]))
        lam = float(rng.choice([0.0, 0.002, 0.01, 0.05, 0.2]))
        tab = orc.decay_table(kind, max(M, K, N), lam)
        A = orc.fill_decay(M, K, tab, int(rng.integers(1, 1000)))
        B = orc.fill_decay(K, N, tab, int(rng.integers(1, 1000)))
        if rng.random() < 0.3:                       # a block of exactly zero tiles
            A[: (M // 2 // tile) * tile, : (K // 2 // tile) * tile] = 0
        dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        ctx.normmap_f32(1, dB, tile)
        ctx.normmap_f32(0, dA, tile)
        q = float(rng.choice([0.0, 0.02, 0.1, 0.5, 1.0]))
        tau = 0.0 if q == 1.0 else (float("inf") if q == 0.0 else ctx.tau_for_ratio(q)[0])
        what = "seed %d case %d: tile %d M %d K %d N %d %s lam %g tau %g" % (seed, case, tile, M, K, N, kind, lam, tau)
        ref = orc.spamm(A, B, tile, tau)
        C = ctx.multiply(dA, dB, tile, tau).clone()
        assert np.array_equal(ctx.get_mask(), ref["mask"]), what
        assert np.array_equal(ctx.get_counts(), ref["counts"]), what
        klist = ctx.get_klist()
        valid = np.arange(klist.shape[2])[None, None, :] < ref["counts"][:, :, None]
        assert np.array_equal(klist[valid], ref["klist"][valid]), what
        assert ctx.get_stats().kept_products == ref["kept"], what
        err, nrm, _ = orc.frob_diff(C.cpu().numpy(), ref["C"])
        assert err <= 1e-3 * nrm, what                               # tolerance of the C parity bar
        assert torch.equal(C, ctx.multiply(dA, dB, tile, tau, prune=True)), what
        assert np.array_equal(ctx.get_mask(), ref["mask"]), what
