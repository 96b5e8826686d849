"""Shape sweep: ragged tile counts, extreme aspect ratios, long k, special values."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
C_REL_TOL = 1e-3


def _dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _check(orc, ctx, A, B, tile, tau):
    import torch
    M, N = A.shape[0], B.shape[1]
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ctx.multiply(_dev(A), _dev(B), tile, tau, C=C)
    ref = orc.spamm(A, B, tile, tau)
    assert np.array_equal(ctx.get_mask(), ref["mask"])
    assert np.array_equal(ctx.get_counts(), ref["counts"])
    assert ctx.get_stats().kept_products == ref["kept"]
    Cg = C.cpu().numpy()
    err, nrm, _ = orc.frob_diff(Cg, ref["C"])
    assert err <= C_REL_TOL * nrm or (nrm == 0 and err == 0)
    return ref


def test_random_shapes(orc, ctx):
    rng = np.random.default_rng(2024)
    for trial in range(40):
        tile = int(rng.choice([32, 64, 128]))
        M, K, N = (int(rng.integers(1, 1 + 1024 // tile)) * tile for _ in range(3))
        lam = float(rng.choice([0.0, 0.005, 0.02, 0.1]))
        tab = orc.decay_table("exp", max(M, K, N), lam)
        A = orc.fill_decay(M, K, tab, 10 + trial)
        B = orc.fill_decay(K, N, tab, 100 + trial)
        nA = orc.normmap(orc.f32_to_f16_bits(A), tile, 0)
        nB = orc.normmap(orc.f32_to_f16_bits(B), tile, 1)
        ratio = float(rng.choice([0.0, 0.1, 0.5, 0.9, 1.0]))
        tau = 0.0 if ratio == 1.0 else (np.inf if ratio == 0.0 else orc.tau_for_ratio(nA, nB, ratio)[0])
        _check(orc, ctx, A, B, tile, tau)


@pytest.mark.parametrize("M,K,N,tile", [(64, 64, 8192, 64), (8192, 64, 64, 64), (64, 16384, 64, 32),
                                        (128, 32768, 128, 128), (2560, 256, 2304, 64), (32, 32, 32, 32),
                                        (288, 32, 2080, 32),
                                        (64, 576, 102400, 64),     # the reference's im2col shape (para.h:20-21)
                                        (32, 288000, 32, 32),      # 9000 k tiles: bitmaps beyond 64 KiB of LDS
                                        (64, 65535 * 64, 64, 64),  # the most k tiles the ABI takes
                                        (32, 65535 * 32, 32, 32)])  # ... at tile 32: the gate walks k in four chunks
def test_extreme_aspect_ratios(orc, ctx, M, K, N, tile):
    tab = orc.decay_table("exp", max(M, K, N), 0.002)
    A = orc.fill_decay(M, K, tab, 1)
    B = orc.fill_decay(K, N, tab, 2)
    nA = orc.normmap(orc.f32_to_f16_bits(A), tile, 0)
    nB = orc.normmap(orc.f32_to_f16_bits(B), tile, 1)
    tau, _ = orc.tau_for_ratio(nA, nB, 0.4)
    ref = _check(orc, ctx, A, B, tile, tau)
    assert 0 < ref["kept"]


@pytest.mark.parametrize("M,n_sup_n,percents", [(256, 520, (100, 40, 10)), (1088, 1030, (100, 30))])
def test_more_than_512_super_tiles_of_c(orc, ctx, M, n_sup_n, percents):
    # beyond 512 super tiles the schedule ranks them by sorting indices padded to a power of two:
    # 1 x 520 -> 1024, and 2 x 1030 = 2060 -> 4096 (M = 1088 is five macro tile rows, the fifth
    # starts a second row of super tiles; 9 GB of C).  B's non-zero column range is cut so that all,
    # 40 % and 10 % of the 520 super tiles hold work -- one case per way of dealing; beyond 2048
    # super tiles there is one way only
    K, tile = 64, 64
    N = n_sup_n * 8 * 256
    tab = orc.decay_table("exp", N, 0.0)
    A = orc.fill_decay(M, K, tab, 1)
    B = orc.fill_decay(K, N, tab, 2)
    for percent in percents:
        cut = N * percent // 100          # a multiple of the tile size
        B[:, cut:] = 0.0
        ref = _check(orc, ctx, A, B, tile, 1e-30)
        assert ref["kept"] == (M // tile) * (cut // tile)


@pytest.mark.parametrize("chunk_words", [1, 3])
def test_gate_in_small_k_chunks_gives_the_same_lists(orc, ctx, chunk_words):
    """A macro tile's bitmaps normally fit a CU's LDS whole; beyond ~19 500 k tiles (tile 32) the
    gate walks k in chunks, twice.  Forcing chunks of 1 and 3 words (64 and 192 k tiles) sends
    ordinary shapes down that path: mask, counts, kept total and C must not change by a bit."""
    import torch
    import cuspamm_amd as sp
    other = sp.SpammContext(0)
    other.set_option(sp.OPT_GATE_CHUNK_WORDS, chunk_words)
    try:
        for (M, K, N), tile, lam, ratio in [((512, 8192, 768), 32, 0.004, 0.3), ((1024, 12800, 512), 64, 0.001, 0.5),
                                            ((256, 33280, 384), 128, 0.0005, 0.4), ((320, 6432, 288), 32, 0.0, 1.0)]:
            tab = orc.decay_table("exp", max(M, K, N), lam)
            dA = torch.empty((M, K), dtype=torch.float32, device="cuda")
            dB = torch.empty((K, N), dtype=torch.float32, device="cuda")
            ctx.fill_decay(dA, tab, 1)
            ctx.fill_decay(dB, tab, 2)
            ctx.normmap_f32(1, dB, tile)
            ctx.normmap_f32(0, dA, tile)
            tau = 0.0 if ratio == 1.0 else ctx.tau_for_ratio(ratio)[0]
            want = ctx.multiply(dA, dB, tile, tau)
            mask, counts, kept = ctx.get_mask(), ctx.get_counts(), ctx.get_stats().kept_products
            got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            other.multiply(dA, dB, tile, tau, C=got)
            assert np.array_equal(other.get_mask(), mask)
            assert np.array_equal(other.get_counts(), counts)
            assert other.get_stats().kept_products == kept and 0 < kept
            assert torch.equal(got, want)
        tab = orc.decay_table("exp", 2048, 0.003)
        _check(orc, other, orc.fill_decay(384, 2048, tab, 3), orc.fill_decay(2048, 320, tab, 4), 32, 0.05)
    finally:
        other.close()


@pytest.mark.parametrize("shape", [2, 3, 4])
def test_other_gemm_work_units_give_the_same_product(orc, ctx, shape):
    """The GEMM's work unit is a whole 256 x 256 macro tile by four waves (shape 1), a 128 x 256
    half by four waves, two workgroups per CU (2), a whole macro tile by eight waves (3), or shape 1
    by workgroups that stay and draw macro tiles from a ticket counter per XCD (4; every case runs
    twice on one gate, so the counter must be back at zero after a launch).  All
    walk the macro tile's list in the same order, so C must agree bit for bit -- whole macro tiles,
    ragged edges where the lower half lies beyond the matrix, all three tile sizes, dense and empty
    regions -- and with the checker."""
    import torch
    import cuspamm_amd as sp
    other = sp.SpammContext(0)
    other.set_option(sp.OPT_GEMM_SHAPE, shape)
    ctx.set_option(sp.OPT_GEMM_SHAPE, 1)
    try:
        for (M, K, N), tile, lam, ratio in [((2304, 1024, 4352), 64, 0.004, 0.3), ((1280, 512, 768), 32, 0.01, 0.5),
                                            ((2048, 2048, 2048), 128, 0.002, 0.2), ((1024, 256, 1280), 64, 0.0, 1.0),
                                            ((384, 2048, 320), 32, 0.003, 0.4), ((128, 1024, 128), 128, 0.0, 1.0),
                                            ((640, 4096, 896), 128, 0.001, 0.1), ((4096, 4096, 4096), 64, 0.01, 0.05),
                                            ((96, 64, 160), 32, 0.0, 1.0)]:
            tab = orc.decay_table("exp", max(M, K, N), lam)
            dA = torch.empty((M, K), dtype=torch.float32, device="cuda")
            dB = torch.empty((K, N), dtype=torch.float32, device="cuda")
            ctx.fill_decay(dA, tab, 1)
            ctx.fill_decay(dB, tab, 2)
            ctx.normmap_f32(1, dB, tile)
            ctx.normmap_f32(0, dA, tile)
            tau = 0.0 if ratio == 1.0 else ctx.tau_for_ratio(ratio)[0]
            want = ctx.multiply(dA, dB, tile, tau)
            mask, kept = ctx.get_mask(), ctx.get_stats().kept_products
            got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            other.multiply(dA, dB, tile, tau, C=got)
            assert np.array_equal(other.get_mask(), mask)
            assert other.get_stats().kept_products == kept and 0 < kept
            assert torch.equal(got, want), (M, K, N, tile)
            got.fill_(float("nan"))
            other.gemm_gated(got)            # the same gate again
            assert torch.equal(got, want), (M, K, N, tile, "second launch on one gate")
        tab = orc.decay_table("exp", 2048, 0.003)
        _check(orc, other, orc.fill_decay(384, 2048, tab, 3), orc.fill_decay(2048, 320, tab, 4), 32, 0.05)
        _check(orc, other, orc.fill_decay(640, 1024, tab, 5), orc.fill_decay(1024, 384, tab, 6), 128, 20.0)
        _check(orc, other, orc.fill_decay(320, 1024, tab, 7), orc.fill_decay(1024, 576, tab, 8), 64, 1.0)
    finally:
        ctx.set_option(sp.OPT_GEMM_SHAPE, 0)
        other.close()


def test_scattered_sparsity_pattern(orc, ctx):
    # no band structure at all: random tiles zeroed, so k lists are ragged and macro tiles mixed
    rng = np.random.default_rng(7)
    n, tile = 1024, 64
    A = rng.uniform(-1, 1, size=(n, n)).astype(np.float32)
    B = rng.uniform(-1, 1, size=(n, n)).astype(np.float32)
    za = rng.random((n // tile, n // tile)) < 0.6
    zb = rng.random((n // tile, n // tile)) < 0.6
    A *= np.kron(~za, np.ones((tile, tile), dtype=np.float32))
    B *= np.kron(~zb, np.ones((tile, tile), dtype=np.float32))
    scale = 10.0 ** rng.integers(-3, 1, size=(n // tile, n // tile))
    A *= np.kron(scale, np.ones((tile, tile))).astype(np.float32)
    ref = _check(orc, ctx, A, B, tile, 1.0)
    assert 0 < ref["kept"] < (n // tile) ** 3 // 2


def test_non_finite_inputs_follow_ieee_compare(orc, ctx):
    # inf tile norm: kept against any non-zero tile; NaN product (inf*0, NaN norm) is dropped
    n, tile = 256, 64
    rng = np.random.default_rng(3)
    A = rng.uniform(-1, 1, size=(n, n)).astype(np.float32)
    B = rng.uniform(-1, 1, size=(n, n)).astype(np.float32)
    A[5, 70] = 1e6            # overflows fp16 -> inf in tile (0,1)
    A[130, 200] = np.nan      # NaN in tile (2,3)
    B[64:128, 0:64] = 0       # zero tile (1,0): inf * 0 = NaN -> dropped
    import torch
    C = torch.empty((n, n), dtype=torch.float32, device="cuda")
    ctx.multiply(_dev(A), _dev(B), tile, 0.5, C=C)
    ref = orc.spamm(A, B, tile, 0.5)
    assert np.array_equal(ctx.get_mask(), ref["mask"])
    assert np.array_equal(ctx.get_counts(), ref["counts"])
    Cg, Cr = C.cpu().numpy(), ref["C"]
    assert np.array_equal(np.isnan(Cg), np.isnan(Cr))
    assert np.array_equal(np.isinf(Cg), np.isinf(Cr))
    fin = np.isfinite(Cr)
    assert np.linalg.norm(Cg[fin] - Cr[fin]) <= C_REL_TOL * np.linalg.norm(Cr[fin])
    assert not ref["mask"][0, 0, 0] & np.uint64(2)      # (i=0, j=0, k=1): inf * 0 is not kept


@pytest.mark.parametrize("n_xcd", [1, 2, 4])
def test_schedule_for_other_xcd_counts_gives_the_same_product(orc, ctx, n_xcd):
    """The GEMM schedule is built for the device's XCD count (8 on a whole MI355X); a partitioned
    device, or one that is not whole XCDs of 32 CUs, gets 4 / 2 / 1 sequences.  The schedule only
    decides where and when a macro tile runs: mask and C must not change by a bit."""
    import torch
    import cuspamm_amd as sp
    other = sp.SpammContext(0)
    other.set_option(sp.OPT_NUM_XCD, n_xcd)
    try:
        # (the last case is a narrow band over 128 super tiles: the grouped row-major deal)
        for (M, K, N), tile, lam, ratio in [((2304, 1024, 4352), 64, 0.004, 0.3), ((1280, 512, 768), 32, 0.01, 0.5),
                                            ((2048, 2048, 2048), 128, 0.002, 0.2), ((8192, 256, 10240), 64, 0.0, 1.0),
                                            ((16384, 16384, 16384), 64, 0.003, 0.1)]:
            tab = orc.decay_table("exp", max(M, K, N), lam)
            dA = torch.empty((M, K), dtype=torch.float32, device="cuda")
            dB = torch.empty((K, N), dtype=torch.float32, device="cuda")
            ctx.fill_decay(dA, tab, 1)
            ctx.fill_decay(dB, tab, 2)
            ctx.normmap_f32(1, dB, tile)
            ctx.normmap_f32(0, dA, tile)
            tau = 0.0 if ratio == 1.0 else ctx.tau_for_ratio(ratio)[0]
            want = ctx.multiply(dA, dB, tile, tau)
            mask = ctx.get_mask()
            got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            other.multiply(dA, dB, tile, tau, C=got)
            assert np.array_equal(other.get_mask(), mask)
            assert torch.equal(got, want)
            del want, got, dA, dB
        tab = orc.decay_table("exp", 1024, 0.01)
        _check(orc, other, orc.fill_decay(768, 1024, tab, 3), orc.fill_decay(1024, 640, tab, 4), 64, 0.3)
    finally:
        other.close()
