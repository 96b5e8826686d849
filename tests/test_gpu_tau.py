"""Device-side tau selection against the host checker (tool.cu:438-490 semantics)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _maps(rng, nbM, nbK, nbN, zero_frac=0.0):
    nA = np.abs(rng.normal(size=(nbM, nbK))).astype(np.float32) * 10 ** rng.uniform(-3, 1, size=(nbM, nbK)).astype(np.float32)
    nB = np.abs(rng.normal(size=(nbK, nbN))).astype(np.float32)
    if zero_frac:
        nA[rng.random(nA.shape) < zero_frac] = 0
    return nA.astype(np.float32), nB.astype(np.float32)


@pytest.mark.parametrize("shape", [(8, 32, 8), (5, 70, 3), (33, 130, 17), (64, 64, 64), (1, 1, 1)])
def test_order_statistic_matches_checker(orc, ctx, shape):
    rng = np.random.default_rng(sum(shape))
    nA, nB = _maps(rng, *shape)
    ctx.set_normmaps(nA, nB, 64)
    for ratio in (0.0, 0.01, 0.1, 0.5, 0.75, 0.999, 1.0):
        tau_g, ach_g = ctx.tau_for_ratio(ratio)
        tau_o, ach_o = orc.tau_for_ratio(nA, nB, ratio)
        assert np.float32(tau_g) == np.float32(tau_o), (ratio, tau_g, tau_o)
        assert ach_g == ach_o
        # and the gate at that tau keeps exactly that many products
        ctx.gate(tau_g)
        assert ctx.get_stats().kept_products == round(ach_g * nA.shape[0] * nA.shape[1] * nB.shape[1])


def test_zero_tail_and_all_zero(orc, ctx):
    rng = np.random.default_rng(1)
    nA, nB = _maps(rng, 16, 48, 16, zero_frac=0.8)
    ctx.set_normmaps(nA, nB, 32)
    for ratio in (0.1, 0.5, 0.9):                              # 0.5 and 0.9 are unreachable with tau > 0
        tau_g, ach_g = ctx.tau_for_ratio(ratio)
        tau_o, ach_o = orc.tau_for_ratio(nA, nB, ratio)
        assert np.float32(tau_g) == np.float32(tau_o) and ach_g == ach_o
        assert tau_g > 0
    ctx.set_normmaps(np.zeros((4, 4), np.float32), np.ones((4, 4), np.float32), 32)
    assert ctx.tau_for_ratio(0.3) == (0.0, 1.0)


def test_count_kept(ctx):
    rng = np.random.default_rng(2)
    nA, nB = _maps(rng, 20, 100, 12)
    ctx.set_normmaps(nA, nB, 64)
    p = (nA[:, None, :] * nB.T[None, :, :]).astype(np.float64)
    for thr in (0.0, 1e-3, 0.5, 7.0):
        cnt, sm = ctx.count_kept(thr)
        assert cnt == int((p >= thr).sum())
        assert abs(sm - p.sum()) <= 1e-9 * p.sum()


def test_reference_bisection(orc, ctx):
    rng = np.random.default_rng(3)
    for shape in [(8, 32, 8), (32, 64, 32)]:
        nA, nB = _maps(rng, *shape)
        ctx.set_normmaps(nA, nB, 32)
        for expected in (0.75, 0.3):
            tau_g, ach_g = ctx.tune_bisect(expected, 0.01, 20)
            tau_o, ach_o = orc.tune_bisect(nA, nB, expected, 0.01, 20)
            assert abs(tau_g - tau_o) <= 1e-6 * abs(tau_o)      # the mean product is summed in another order
            assert abs(ach_g - ach_o) <= 2.0 / (shape[0] * shape[1] * shape[2])
            assert abs(ach_g - expected) < 0.01


def test_bisection_iterates_match_the_hand_worked_sequence(ctx):
    # the sequences worked by hand from tool.cu:445-486 (products 1, 2, 3, 4; all sums exact)
    from test_oracle_gate import BISECT_HAND
    ctx.set_normmaps(np.array([[1.0, 2.0, 3.0, 4.0]], dtype=np.float32), np.ones((4, 1), dtype=np.float32), 32)
    for expected, seq in BISECT_HAND.items():
        for rounds, want in enumerate(seq, start=1):
            assert ctx.tune_bisect(expected, 0.01, rounds) == want, (expected, rounds)
    assert ctx.tune_bisect(0.25, 0.01, 20) == (3.75, 0.25)
    assert ctx.tune_bisect(0.75, 0.01, 20) == (1.25, 0.75)


def test_dropped_bound_hand_worked(ctx):
    # per output tile the dropped products sum to 7, 10, 4, 8 at tau = 10 and to 7, 2, 4, 0 at
    # tau = 8 (a product equal to tau is kept)
    nA = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.float32)
    nB = np.array([[1, 2], [3, 4], [5, 6]], dtype=np.float32)
    ctx.set_normmaps(nA, nB, 32)
    assert ctx.dropped_bound(10.0) == pytest.approx(np.sqrt(229.0), rel=1e-14)
    assert ctx.dropped_bound(8.0) == pytest.approx(np.sqrt(69.0), rel=1e-14)
    assert ctx.dropped_bound(0.0) == 0.0


def test_full_size_selection(orc, ctx):
    import torch
    N, tile = 16384, 64
    tab = orc.decay_table("exp", N, 0.003)
    dA = torch.empty((N, N), dtype=torch.float32, device="cuda")
    dB = torch.empty((N, N), dtype=torch.float32, device="cuda")
    ctx.fill_decay(dA, tab, 1)
    ctx.fill_decay(dB, tab, 2)
    ctx.normmap_f32(1, dB, tile)
    ctx.normmap_f32(0, dA, tile)
    tau_g, ach_g = ctx.tau_for_ratio(0.10)
    tau_o, ach_o = orc.tau_for_ratio(ctx.get_normmap(0), ctx.get_normmap(1), 0.10)
    assert np.float32(tau_g) == np.float32(tau_o) and ach_g == ach_o
    assert abs(ach_g - 0.10) < 1e-4
